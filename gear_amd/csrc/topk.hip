// Top-k of fp32 priorities by radix select + ordered compaction + radix sort, gfx950.
//
// fp32 priorities map to order-preserving uint32 keys.  Three histogram passes (11 + 11 + 10
// bits, LDS histograms, the consuming launch picks the bin) find the key T of the k-th largest
// priority and how many entries equal to T are still needed.  An ordered compaction in two
// launches writes the selected entries in index order: every entry above T, and the first need_eq
// entries equal to T -- ties go to the smaller index.  The count launch also lists every wave's
// candidates (entries >= T), so the write launch touches only those; where the maxima are
// clustered a list overflows and the write launch re-reads the priorities instead.  For value
// order the k candidates then go through the stable LSD radix sort on the inverted key.
// The streaming loops are sensitive to their instruction count (a launch that reads 40 MB spends
// as long issuing ~10 instructions per element as waiting for memory), so they compare floats
// (one instruction, same order as the keys for non-NaN values) wherever a key is not needed.
#include "radix_sort.hpp"

namespace gearhip {
namespace {

constexpr int kBlock = 256;
constexpr int kMaxRanges = 2048;  // workgroups of the compaction launches
constexpr int kCompactThreads = 512;  // threads of a compaction workgroup (256: +2.5 us at n = 1e7)
constexpr int kWavesPerBlock = kCompactThreads / kWave;
constexpr int kHistBins = 2048;
// Histogram launches: one 1024-thread workgroup per CU.  Fewer, fatter workgroups mean fewer
// flush atomics per bin and fewer workgroups that pick the previous bin (measured at n = 1e7:
// 512 x 256 threads 60.8 us for the whole top-k, 256 x 512 56.0, 512 x 1024 54.9, 256 x 1024 53.1).
constexpr int kMaxHistBlocks = 256;
constexpr int kHistThreads = 1024;

struct State {
  uint32_t prefix[3];  // key bits decided after pass 0, 1, 2 (right-aligned)
  uint32_t k_rem[3];   // entries still to take from the bin picked in that pass
  uint32_t overflow;   // a wave found more candidates than its list holds: the write launch re-reads
  uint32_t pad[57];
};
static_assert(sizeof(State) == 256, "State is the 256-byte header of the workspace");

__device__ __forceinline__ uint32_t order_key(float f) {
  const uint32_t b = __float_as_uint(f);
  // positive: set the sign bit; negative: flip every bit
  uint32_t key = b ^ ((uint32_t)((int32_t)b >> 31) | 0x80000000u);
  key += key == 0x7fffffffu ? 1u : 0u;  // -0.0 ranks with +0.0
  return key;
}

constexpr int kStep = kWave * 4;  // elements one wave handles per step (one float4 per lane)
constexpr int kAhead = 4;         // steps whose loads are in flight together

// Geometry of the compaction launches: `ranges` workgroups, every wave owns wave_len consecutive
// elements (a multiple of kStep) and a candidate list of list_cap entries.
struct Geom {
  int64_t ranges, wave_len, list_cap;
};

Geom geom(int64_t n, int64_t k) {
  Geom g;
  g.ranges = ceil_div64(n > 0 ? n : 1, (int64_t)kWavesPerBlock * kAhead * kStep);
  if (g.ranges > kMaxRanges) g.ranges = kMaxRanges;
  g.wave_len = ceil_div64(ceil_div64(n > 0 ? n : 1, g.ranges * kWavesPerBlock), kStep) * kStep;
  g.ranges = ceil_div64(n > 0 ? n : 1, g.wave_len * kWavesPerBlock);
  // four times a wave's fair share of the k selected entries, at least 64, never more than the
  // wave has elements; clustered maxima or many ties overflow it and take the re-reading path
  const int64_t waves = g.ranges * kWavesPerBlock;
  int64_t cap = ceil_div64(4 * ceil_div64(k > 0 ? k : 1, waves), 64) * 64;
  if (cap < 64) cap = 64;
  if (cap > g.wave_len) cap = g.wave_len;
  g.list_cap = cap;
  return g;
}

// the priority whose order_key is `key` (for +-0.0: +0.0)
__device__ __forceinline__ float key_to_float(uint32_t key) {
  return __uint_as_float((key & 0x80000000u) ? (key ^ 0x80000000u) : ~key);
}

struct Layout {
  size_t hist, desc, lists, ckey, cidx, skey, sidx, tkey, tidx, shist, total;
};

Layout layout(int64_t n, int64_t k) {
  Layout l;
  const size_t kk = align_up((size_t)(k > 0 ? k : 1) * 4, 256);
  const Geom g = geom(n, k);
  size_t o = sizeof(State);
  l.hist = o;  o += 3 * kHistBins * sizeof(uint32_t);
  l.desc = o;  o += (size_t)kMaxRanges * (kWavesPerBlock + 1) * 8;  // wave and workgroup counts
  l.lists = o; o += align_up((size_t)(g.ranges * kWavesPerBlock * g.list_cap) * 4, 256);
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
template <int PASS, int THREADS = kBlock>
__device__ __forceinline__ Pick pick_bin(int64_t k, State *state, const uint32_t *hist) {
  constexpr int kBinsHere = PASS == 2 ? 1024 : 2048;
  constexpr int kPerThread = kBinsHere / THREADS;
  __shared__ uint32_t wsum[THREADS / kWave];
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
  // fallback when no bin holds the k_rem-th key (only possible with NaN priorities, which the
  // float compares of the later passes do not count): the lowest bin, nothing taken off k_rem
  if (tid == 0) {
    s_pick.prefix = PASS == 0 ? 0u : (PASS == 1 ? (prefix << 11) : (prefix << 10));
    s_pick.k_rem = k_rem;
  }
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
__global__ __launch_bounds__(kHistThreads) void select_hist_kernel(const float *__restrict__ p,
                                                             int64_t n, int64_t k, State *state,
                                                             uint32_t *hist) {
  constexpr int kBinsHere = PASS == 2 ? 1024 : 2048;
  typedef float f4 __attribute__((ext_vector_type(4), aligned(4)));
  __shared__ uint32_t h[kBinsHere];
  const int tid = threadIdx.x;
  for (int i = tid; i < kBinsHere; i += kHistThreads) h[i] = 0;
  uint32_t prefix = 0u;
  if (PASS == 1) prefix = pick_bin<0, kHistThreads>(k, state, hist - kHistBins).prefix;
  if (PASS == 2) prefix = pick_bin<1, kHistThreads>(k, state, hist - kHistBins).prefix;
  __syncthreads();

  // Passes 1 and 2 count only the keys that start with `prefix`: about 1 % of the input.  Whether
  // a priority is one of them is decided with two float compares against the bounds of that key
  // range (float order = key order for non-NaN values, -0.0 == +0.0); the key itself is worked
  // out only for the members.
  constexpr int kLowBits = PASS == 1 ? 21 : 10;
  uint32_t lo_key = PASS == 0 ? 0u : prefix << kLowBits;
  uint32_t hi_key = PASS == 0 ? 0u : (lo_key | ((1u << kLowBits) - 1u));
  if (hi_key == 0x7fffffffu) hi_key = 0x7ffffffeu;  // the key below +-0.0's: the zeros are not in this range
  // the bins that hold +inf / -inf reach into keys that decode to NaN, with which every compare
  // is false: the bounds stop at the keys of the infinities
  constexpr uint32_t kKeyPosInf = 0xff800000u, kKeyNegInf = 0x007fffffu;
  if (hi_key > kKeyPosInf) hi_key = kKeyPosInf;
  if (lo_key < kKeyNegInf) lo_key = kKeyNegInf;
  const float lo_f = key_to_float(lo_key), hi_f = key_to_float(hi_key);
  auto count = [&](float f) {
    if (PASS == 0) {
      atomicAdd(&h[order_key(f) >> 21], 1u);
    } else if (f >= lo_f && f <= hi_f) {
      const uint32_t key = order_key(f);
      atomicAdd(&h[PASS == 1 ? ((key >> 10) & 0x7ffu) : (key & 0x3ffu)], 1u);
    }
  };
  const int64_t nvec = n >> 2;
  constexpr int kLoads = 4;  // 16-byte loads in flight per thread
  for (int64_t v0 = (int64_t)blockIdx.x * kHistThreads * kLoads + tid; v0 < nvec;
       v0 += (int64_t)gridDim.x * kHistThreads * kLoads) {
    f4 q[kLoads];
#pragma unroll
    for (int u = 0; u < kLoads; ++u) {
      const int64_t v = v0 + (int64_t)u * kHistThreads;
      q[u] = f4{0.0f, 0.0f, 0.0f, 0.0f};
      if (v < nvec) q[u] = *reinterpret_cast<const f4 *>(p + (v << 2));
    }
#pragma unroll
    for (int u = 0; u < kLoads; ++u) {
      if (v0 + (int64_t)u * kHistThreads < nvec) {
        count(q[u][0]);
        count(q[u][1]);
        count(q[u][2]);
        count(q[u][3]);
      }
    }
  }
  if (blockIdx.x == 0 && tid < (int)(n & 3)) count(p[(nvec << 2) + tid]);
  __syncthreads();
  for (int i = tid; i < kBinsHere; i += kHistThreads)
    if (h[i]) atomicAdd(&hist[i], h[i]);
}

// Ordered compaction in two launches with no waiting between workgroups.  The input is cut into
// gridDim.x * 4 contiguous wave ranges of wave_len elements (a multiple of kStep).  The count
// launch writes every wave's packed (greater << 31 | equal) count and every workgroup's total; the
// write launch sums the totals of the workgroups before it, adds the counts of the waves before it
// in its own workgroup, and walks its range again (now from L2 / MALL) placing the selected entries.
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

__global__ __launch_bounds__(kCompactThreads) void count_ranges_kernel(
    const float *__restrict__ p, int64_t n, int64_t k, State *state, const uint32_t *hist2,
    int64_t wave_len, uint64_t *__restrict__ wave_counts, uint64_t *__restrict__ block_counts,
    uint32_t *__restrict__ lists, int list_cap) {
  __shared__ int64_t red[kWavesPerBlock];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t gw = (int64_t)blockIdx.x * kWavesPerBlock + wave;
  const int64_t begin = gw * wave_len;
  const int64_t end = begin + wave_len < n ? begin + wave_len : n;
  uint32_t *list = lists + gw * list_cap;
  const uint64_t lt_mask = lane == 0 ? 0ull : (~0ull >> (64 - lane));
  int listed = 0;         // candidates of this wave so far (wave-uniform)
  bool overflow = false;  // wave-uniform
  // the first loads are issued before the threshold is picked so that the two latencies overlap
  float q[kAhead][4];
#pragma unroll
  for (int a = 0; a < kAhead; ++a) load_quad(p, begin + (int64_t)a * kStep + lane * 4, end, q[a]);
  const float thr_f = key_to_float(pick_bin<2, kCompactThreads>(k, state, hist2).prefix);
  uint32_t gt = 0, eq = 0;
  for (int64_t s0 = begin; s0 < end; s0 += kAhead * kStep) {
    // the next batch of loads is in flight while this one is classified and listed
    float qn[kAhead][4];
    const int64_t s1 = s0 + kAhead * kStep;
    if (s1 < end) {
#pragma unroll
      for (int a = 0; a < kAhead; ++a) load_quad(p, s1 + (int64_t)a * kStep + lane * 4, end, qn[a]);
    }
#pragma unroll
    for (int a = 0; a < kAhead; ++a) {
      const int64_t e0 = s0 + (int64_t)a * kStep + lane * 4;
      // every candidate (greater than, or equal to, the threshold) goes to the wave's list in
      // index order as index | greater << 31; the write launch then never reads the priorities
      bool sel[4];
      uint32_t val[4];
      int off[4], nc = 0;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        // float compares order non-NaN priorities exactly like their keys (-0.0 == +0.0) at
        // one instruction each
        const bool above = q[a][j] > thr_f;
        sel[j] = e0 + j < end && q[a][j] >= thr_f;
        off[j] = nc;
        nc += sel[j] ? 1 : 0;
        gt += sel[j] && above;
        eq += sel[j] && !above;
        val[j] = (uint32_t)(e0 + j) | (above ? 0x80000000u : 0u);
      }
      if (wave_ballot(nc != 0) == 0ull) continue;
      // candidates in the lanes before this one: nc <= 4 is three bits, one ballot per bit
      // (independent instructions; a DPP scan is a chain of a dozen dependent ones)
      const uint64_t b0 = wave_ballot((nc & 1) != 0), b1 = wave_ballot((nc & 2) != 0),
                     b2 = wave_ballot((nc & 4) != 0);
      const int before = __popcll(b0 & lt_mask) + 2 * __popcll(b1 & lt_mask) +
                         4 * __popcll(b2 & lt_mask);
      const int total = __popcll(b0) + 2 * __popcll(b1) + 4 * __popcll(b2);
      if (listed + total > list_cap) {
        overflow = true;
      } else {
        const int at = listed + before;
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (sel[j]) list[at + off[j]] = val[j];
      }
      listed += total;
    }
#pragma unroll
    for (int a = 0; a < kAhead; ++a)
#pragma unroll
      for (int j = 0; j < 4; ++j) q[a][j] = qn[a][j];
  }
  if (overflow && lane == 0) state->overflow = 1u;  // same value from every overflowing wave
  const int64_t w = wave_sum(((int64_t)gt << 31) | (int64_t)eq);
  if (lane == 0) {
    wave_counts[gw] = (uint64_t)w;
    red[wave] = w;
  }
  __syncthreads();
  if (tid == 0) {
    int64_t t = 0;
#pragma unroll
    for (int i = 0; i < kWavesPerBlock; ++i) t += red[i];
    block_counts[blockIdx.x] = (uint64_t)t;
  }
}

template <bool DIRECT>
__global__ __launch_bounds__(kCompactThreads) void write_ranges_kernel(
    const float *__restrict__ p, int64_t n, int64_t k, const State *state, int64_t wave_len,
    const uint64_t *__restrict__ wave_counts, const uint64_t *__restrict__ block_counts,
    const uint32_t *__restrict__ lists, int list_cap, uint32_t *__restrict__ ckey,
    uint32_t *__restrict__ cidx, float *__restrict__ values_out,
    int64_t *__restrict__ indices_out) {
  __shared__ int64_t red[kWavesPerBlock];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t gw = (int64_t)blockIdx.x * kWavesPerBlock + wave;
  const int64_t begin = gw * wave_len;
  const int64_t end = begin + wave_len < n ? begin + wave_len : n;
  const bool reread = state->overflow != 0u;  // some wave's list was too short: all waves re-read
  float q[kAhead][4];
  if (reread) {
#pragma unroll
    for (int a = 0; a < kAhead; ++a) load_quad(p, begin + (int64_t)a * kStep + lane * 4, end, q[a]);
  }
  const float thr_f = key_to_float(state->prefix[2]);
  const uint32_t need_eq = state->k_rem[2];

  int64_t part = 0;
  for (int j = tid; j < (int)blockIdx.x; j += kCompactThreads) part += (int64_t)block_counts[j];
  const int64_t pw = wave_sum(part);
  if (lane == 0) red[wave] = pw;
  __syncthreads();
  int64_t excl = 0;
#pragma unroll
  for (int i = 0; i < kWavesPerBlock; ++i) excl += red[i];
  // plus the waves before this one in its own workgroup
  int64_t own = 0;
  if (lane < wave) own = (int64_t)wave_counts[(int64_t)blockIdx.x * kWavesPerBlock + lane];
  excl += wave_sum(own);
  uint32_t gt_run = (uint32_t)(excl >> 31), eq_run = (uint32_t)(excl & 0x7fffffff);

  auto emit = [&](uint32_t pos, int64_t index, float value, uint32_t key) {
    if (pos >= (uint32_t)k) return;  // counts that NaN priorities put out of step never leave the outputs
    if (DIRECT) {
      indices_out[pos] = index;
      if (values_out) values_out[pos] = value;
    } else {
      ckey[pos] = ~key;
      cidx[pos] = (uint32_t)index;
    }
  };

  if (!reread) {
    // the wave's candidates, in index order, from its list
    const uint64_t mine = wave_counts[gw];
    const int m = (int)(mine >> 31) + (int)(mine & 0x7fffffff);
    const uint32_t *list = lists + gw * list_cap;
    const uint64_t lt_mask = lane == 0 ? 0ull : (~0ull >> (64 - lane));
    for (int c0 = 0; c0 < m; c0 += kWave) {
      const bool valid = c0 + lane < m;
      const uint32_t ent = valid ? list[c0 + lane] : 0u;
      const bool is_gt = valid && (ent >> 31) != 0u, is_eq = valid && (ent >> 31) == 0u;
      const uint64_t bg = wave_ballot(is_gt), be = wave_ballot(is_eq);
      const uint32_t g = gt_run + (uint32_t)__popcll(bg & lt_mask);
      const uint32_t e = eq_run + (uint32_t)__popcll(be & lt_mask);
      if (is_gt || (is_eq && e < need_eq)) {
        const uint32_t index = ent & 0x7fffffffu;
        const float value = p[index];
        emit(g + (e < need_eq ? e : need_eq), (int64_t)index, value, order_key(value));
      }
      gt_run += (uint32_t)__popcll(bg);
      eq_run += (uint32_t)__popcll(be);
    }
    return;
  }

  for (int64_t s0 = begin; s0 < end; s0 += kAhead * kStep) {
    if (s0 != begin) {
#pragma unroll
      for (int a = 0; a < kAhead; ++a) load_quad(p, s0 + (int64_t)a * kStep + lane * 4, end, q[a]);
    }
#pragma unroll
    for (int a = 0; a < kAhead; ++a) {
      const int64_t e0 = s0 + (int64_t)a * kStep + lane * 4;
      int s = 0;  // packed counts of the lane's four entries: greater << 16 | equal
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (e0 + j < end) s += q[a][j] > thr_f ? (1 << 16) : (q[a][j] == thr_f ? 1 : 0);
      if (wave_ballot(s != 0) == 0ull) continue;
      const int inc = wave_inclusive_sum(s);
      const int total = wave_read_lane(inc, kWave - 1);
      const int before = inc - s;
      uint32_t g = gt_run + ((uint32_t)before >> 16);
      uint32_t e = eq_run + ((uint32_t)before & 0xffffu);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (e0 + j < end) {
          const bool is_gt = q[a][j] > thr_f, is_eq = q[a][j] == thr_f;
          if (is_gt || (is_eq && e < need_eq))
            emit(g + (e < need_eq ? e : need_eq), e0 + j, q[a][j], order_key(q[a][j]));
          g += is_gt;
          e += is_eq;
        }
      }
      gt_run += (uint32_t)total >> 16;
      eq_run += (uint32_t)total & 0xffffu;
    }
  }
}

// Final store of the value-ordered form, fused into the last digit of the candidate sort.
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

__global__ __launch_bounds__(kBlock) void emit_kernel(const float *__restrict__ p,
                                                      const uint32_t *__restrict__ sidx, int64_t k,
                                                      int64_t n, float *__restrict__ values_out,
                                                      int64_t *__restrict__ indices_out) {
  const int64_t j = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (j >= k) return;
  const uint32_t i = sidx[j];
  indices_out[j] = (int64_t)i;
  if (values_out) values_out[j] = (int64_t)i < n ? p[i] : 0.0f;
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
  hipStream_t st = as_stream(stream);

  const int64_t zero_words = (int64_t)(l.desc / 4);  // header + histograms
  zero_kernel<<<dim3((unsigned)ceil_div64(zero_words, 256)), dim3(256), 0, st>>>(
      reinterpret_cast<uint32_t *>(ws), zero_words);
  int64_t hblocks = ceil_div64(n, (int64_t)kHistThreads * 4 * 4);
  if (hblocks < 1) hblocks = 1;
  if (hblocks > kMaxHistBlocks) hblocks = kMaxHistBlocks;
  const dim3 hgrid((unsigned)hblocks), hblock(kHistThreads), block(kBlock);
  select_hist_kernel<0><<<hgrid, hblock, 0, st>>>(priorities, n, k, state, hist);
  select_hist_kernel<1><<<hgrid, hblock, 0, st>>>(priorities, n, k, state, hist + kHistBins);
  select_hist_kernel<2><<<hgrid, hblock, 0, st>>>(priorities, n, k, state, hist + 2 * kHistBins);
  GEARHIP_RETURN_IF_LAUNCH_FAILED();

  uint32_t *ckey = reinterpret_cast<uint32_t *>(ws + l.ckey);
  uint32_t *cidx = reinterpret_cast<uint32_t *>(ws + l.cidx);
  const bool direct = !sorted_by_value;
  const Geom g = geom(n, k);
  const int64_t ranges = g.ranges, wave_len = g.wave_len;
  uint32_t *lists = reinterpret_cast<uint32_t *>(ws + l.lists);
  uint64_t *wave_counts = reinterpret_cast<uint64_t *>(ws + l.desc);
  uint64_t *block_counts = wave_counts + (size_t)kMaxRanges * kWavesPerBlock;
  const dim3 cgrid((unsigned)ranges), cblock(kCompactThreads);
  count_ranges_kernel<<<cgrid, cblock, 0, st>>>(priorities, n, k, state, hist + 2 * kHistBins,
                                               wave_len, wave_counts, block_counts, lists,
                                               (int)g.list_cap);
  if (direct)
    write_ranges_kernel<true><<<cgrid, cblock, 0, st>>>(priorities, n, k, state, wave_len, wave_counts,
                                                       block_counts, lists, (int)g.list_cap, ckey,
                                                       cidx, values_out, indices_out);
  else
    write_ranges_kernel<false><<<cgrid, cblock, 0, st>>>(priorities, n, k, state, wave_len,
                                                        wave_counts, block_counts, lists,
                                                        (int)g.list_cap, ckey, cidx, values_out,
                                                        indices_out);
  GEARHIP_RETURN_IF_LAUNCH_FAILED();
  if (direct) return 0;
  uint32_t *skey = reinterpret_cast<uint32_t *>(ws + l.skey);
  uint32_t *sidx = reinterpret_cast<uint32_t *>(ws + l.sidx);
  uint32_t *tkey = reinterpret_cast<uint32_t *>(ws + l.tkey);
  uint32_t *tidx = reinterpret_cast<uint32_t *>(ws + l.tidx);
  uint32_t *shist = reinterpret_cast<uint32_t *>(ws + l.shist);
  if (k > radix::kRankMax) {
    // radix path: the last digit's scatter writes values_out / indices_out itself
    const EmitSorted fin{priorities, values_out, indices_out, (uint32_t)n};
    return radix::sort_pairs<uint32_t, uint32_t, EmitSorted>(ckey, skey, cidx, sidx, tkey, tidx, k,
                                                             0, 32, shist, st, fin);
  }
  int rc = radix::sort_pairs<uint32_t, uint32_t>(ckey, skey, cidx, sidx, tkey, tidx, k, 0, 32,
                                                 shist, st);
  if (rc) return rc;
  emit_kernel<<<dim3((unsigned)ceil_div64(k, kBlock)), block, 0, st>>>(priorities, sidx, k, n,
                                                                      values_out, indices_out);
  GEARHIP_RETURN_IF_LAUNCH_FAILED();
  return 0;
}
