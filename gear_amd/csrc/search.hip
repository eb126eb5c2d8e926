// Batched upper_bound of draws in an inclusive prefix array (+ importance weights), and the
// one-call batch sampler (search + ranking sort + split into window arguments), gfx950.
//
// One thread per draw, one wave per workgroup.  The first levels of the search touch the same few
// prefix entries for every draw, so they are served by the caches; the search is latency-bound
// (a chain of log8(n) + 1 dependent load steps), which is why all draws of a batch run concurrently
// and spread over many CUs.
#include <math.h>

#include "radix_sort.hpp"

namespace gearhip {
namespace {

constexpr int kBlock = 256;
constexpr int kSearchBlock = 64;  // one wave per workgroup: spreads the divergent probes over many CUs

// First index with p[i] > t (n when there is none).  The search is kArity-ary: kArity - 1
// independent probes per step cut the chain of dependent loads from log2(n) to log_kArity(n)
// steps, and the chain, not the number of loads, is what a batch of draws waits for.  The last
// step reads the whole remaining stretch at once.
constexpr int kArity = 8;  // 16 probes per step measured slower (4.5 against 4.05 us at n = 1e6)
constexpr int kArityShift = 3;

template <typename T>
__device__ __forceinline__ int64_t upper_bound_dev(const T *__restrict__ p, int64_t n, T t) {
  int64_t lo = 0, hi = n;  // the answer lies in [lo, hi]
  while (hi - lo >= kArity) {
    const int64_t step = (hi - lo) >> kArityShift;
    T v[kArity - 1];
#pragma unroll
    for (int j = 0; j < kArity - 1; ++j) v[j] = p[lo + step * (j + 1) - 1];
    int c = 0;  // probes are ordered, so the ones <= t form a prefix
#pragma unroll
    for (int j = 0; j < kArity - 1; ++j) c += (v[j] <= t) ? 1 : 0;
    const int64_t base = lo + step * c;
    if (c < kArity - 1) hi = lo + step * (c + 1) - 1;
    lo = base;
  }
  // fewer than kArity candidates left: p[lo .. hi) in one go (entries are ordered)
  T v[kArity - 1];
#pragma unroll
  for (int j = 0; j < kArity - 1; ++j) v[j] = lo + j < hi ? p[lo + j] : t;
  int c = 0;
#pragma unroll
  for (int j = 0; j < kArity - 1; ++j) c += (lo + j < hi && v[j] <= t) ? 1 : 0;
  return lo + c;
}

__global__ __launch_bounds__(kSearchBlock) void search_f64_kernel(
    const double *__restrict__ prefix, int64_t n, const float *__restrict__ u, int64_t num,
    int unit, int64_t *__restrict__ idx_out, const float *__restrict__ priorities, double beta,
    double *__restrict__ wraw, double *__restrict__ block_max) {
  const int64_t j = (int64_t)blockIdx.x * kSearchBlock + threadIdx.x;
  const double total = prefix[n - 1];
  double w = 0.0;
  if (j < num) {
    const double t = unit ? (double)u[j] * total : (double)u[j];
    int64_t i = upper_bound_dev<double>(prefix, n, t);
    if (i > n - 1) i = n - 1;
    idx_out[j] = i;
    if (priorities != nullptr) {
      w = pow((double)n * (double)priorities[i] / total, -beta);
      wraw[j] = w;
    }
  }
  if (priorities != nullptr) {
    // workgroup (= wave) maximum of the raw weights (weights are positive, padding lanes hold 0)
    double m = w;
    for (int off = 32; off > 0; off >>= 1) m = fmax(m, __shfl_xor(m, off, kWave));
    if (threadIdx.x == 0) block_max[blockIdx.x] = m;
  }
}

__global__ __launch_bounds__(kBlock) void normalise_kernel(const double *__restrict__ wraw,
                                                           const double *__restrict__ block_max,
                                                           int nblocks, int64_t num,
                                                           float *__restrict__ out) {
  __shared__ double wmax[kBlock / kWave];
  double m = 0.0;
  for (int i = threadIdx.x; i < nblocks; i += kBlock) m = fmax(m, block_max[i]);
  for (int off = 32; off > 0; off >>= 1) m = fmax(m, __shfl_xor(m, off, kWave));
  if ((threadIdx.x & 63) == 0) wmax[threadIdx.x >> 6] = m;
  __syncthreads();
  m = fmax(fmax(wmax[0], wmax[1]), fmax(wmax[2], wmax[3]));
  const int64_t j = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (j < num) out[j] = (float)(wraw[j] / m);
}

// The draw of an int64 prefix (a sampler over lengths): u holds doubles in [0, 1) (unit) or
// int64 targets.
struct DrawI64 {
  const int64_t *prefix;
  int64_t n;
  const void *u;
  int unit;
  __device__ __forceinline__ int64_t operator()(int64_t j) const {
    const int64_t total = prefix[n - 1];
    int64_t t;
    if (unit)
      t = (int64_t)floor(static_cast<const double *>(u)[j] * (double)total);
    else
      t = static_cast<const int64_t *>(u)[j];
    const int64_t i = upper_bound_dev<int64_t>(prefix, n, t);
    return i > n - 1 ? n - 1 : i;
  }
};
__global__ __launch_bounds__(kSearchBlock) void search_i64_kernel(DrawI64 draw, int64_t num,
                                                                  int64_t *__restrict__ idx_out) {
  const int64_t j = (int64_t)blockIdx.x * kSearchBlock + threadIdx.x;
  if (j < num) idx_out[j] = draw(j);
}

// The ranking sort of radix_sort.hpp over the found indices, fused with the split into window
// arguments.  Used for prefixes shorter than 2^32 entries (the compare key is the index as
// uint32_t); longer ones take the radix sort.
struct Split {
  int64_t *sorted_out;
  int64_t T, modulo;
  int64_t *idxs, *tss, *lens;
  // the entry at sorted place `rank` is the flat index `mine` (below 2^32)
  __device__ __forceinline__ void operator()(int64_t rank, int64_t f) const {
    const uint32_t mine = (uint32_t)f;
    if (sorted_out) sorted_out[rank] = f;
    if (T > 0) {
      int64_t traj, ts;
      if (T <= 0xffffffffll && modulo <= 0xffffffffll) {
        uint32_t f32 = mine;  // 32-bit division is a fraction of the 64-bit one
        if (modulo > 0) f32 %= (uint32_t)modulo;
        const uint32_t q = f32 / (uint32_t)T;
        traj = q;
        ts = f32 - q * (uint32_t)T;
      } else {
        if (modulo > 0) f %= modulo;
        traj = f / T;
        ts = f - traj * T;
      }
      idxs[rank] = traj;
      tss[rank] = ts;
      if (lens) lens[rank] = ts + 1;
    }
  }
};

__global__ __launch_bounds__(radix::kRankBlock) void rank_split_kernel(
    const int64_t *__restrict__ raw, int num, Split split) {
  typedef uint32_t K;
  __shared__ radix::RankSmem<K> sm;
  K mine;
  const uint32_t rank = radix::block_rank<K>(sm, num, [&](int j) { return (K)raw[j]; }, &mine);
  const int e = (int)blockIdx.x * kWave + (threadIdx.x & 63);
  if (threadIdx.x >= kWave || e >= num) return;
  split((int64_t)rank, (int64_t)mine);
}

__global__ __launch_bounds__(kBlock) void split_sorted_kernel(const int64_t *__restrict__ flat,
                                                              int64_t num, int64_t T,
                                                              int64_t modulo,
                                                              int64_t *__restrict__ idxs,
                                                              int64_t *__restrict__ tss,
                                                              int64_t *__restrict__ lens) {
  const int64_t j = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (j >= num) return;
  int64_t f = flat[j];
  if (modulo > 0) f %= modulo;
  const int64_t traj = f / T;
  const int64_t ts = f - traj * T;
  idxs[j] = traj;
  tss[j] = ts;
  if (lens) lens[j] = ts + 1;
}

// What the loader does with a sorted batch of positions before it can gather
// (gear/loader/offline_loader.py:168-177 and the samplers' concat_indices[draws],
// gear/sampler/global_sampler.py:131,172,196), for the entry at sorted place r with position p:
//     sampled[r] = index_table ? index_table[p] : p        the batch's global trajectory index
//     local[r]   = sampled[r] - index_offset               its index in this shard's table
//     lens[r]    = lengths_table[local[r]]                  its recorded length (0 outside the table)
struct Lookup {
  const int64_t *index_table;
  int64_t index_n, index_offset;
  const int64_t *lengths_table;
  int64_t lengths_n;
  int64_t *sampled, *local, *lens;
  // a window of `window` steps inside the entry's recorded length, placed by a uniform:
  // starts[r] = floor(start_u[r] * (length - window + 1)), 0 for a length below the window
  const double *start_u = nullptr;
  int64_t window = 0;
  int64_t *starts = nullptr;
  __device__ __forceinline__ void operator()(int64_t r, int64_t p) const {
    int64_t g = p;
    if (index_table) g = (p >= 0 && p < index_n) ? index_table[p] : 0;
    const int64_t l = g - index_offset;
    if (sampled) sampled[r] = g;
    if (local) local[r] = l;
    const int64_t len = (lengths_table && l >= 0 && l < lengths_n) ? lengths_table[l] : 0;
    if (lens) lens[r] = len;
    if (starts) {
      const int64_t room = len - (window - 1);
      starts[r] = room > 0 ? (int64_t)floor(start_u[r] * (double)room) : 0;
    }
  }
};

// The ranking sort over a batch of positions (at most kRankMax, each below 2^32), with the
// look-ups of the sorted entry done by the thread that ranked it: one launch instead of a sort
// and two gathers.
__global__ __launch_bounds__(radix::kRankBlock) void rank_lookup_kernel(
    const int64_t *__restrict__ raw, int num, Lookup look) {
  typedef uint32_t K;
  __shared__ radix::RankSmem<K> sm;
  K mine;
  const uint32_t rank = radix::block_rank<K>(sm, num, [&](int j) { return (K)raw[j]; }, &mine);
  const int e = (int)blockIdx.x * kWave + (threadIdx.x & 63);
  if (threadIdx.x >= kWave || e >= num) return;
  look((int64_t)rank, (int64_t)mine);
}

__global__ __launch_bounds__(kBlock) void lookup_kernel(const int64_t *__restrict__ positions,
                                                        int64_t num, Lookup look) {
  const int64_t j = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (j < num) look(j, positions[j]);
}

struct SampleWs {
  size_t raw, ktmp, sorted, hist, total;
};
SampleWs sample_ws(int64_t num) {
  SampleWs w;
  const size_t m = align_up((size_t)(num > 0 ? num : 1) * 8, 256);
  w.raw = 0;
  w.ktmp = m;
  w.sorted = 2 * m;
  w.hist = 3 * m;
  w.total = 3 * m + radix::hist_bytes(num);
  return w;
}

size_t search_ws_bytes(int64_t num) {
  if (num <= 0) return 256;
  const int64_t blocks = ceil_div64(num, kSearchBlock);
  return align_up((size_t)num * 8, 256) + align_up((size_t)blocks * 8, 256);
}

}  // namespace
}  // namespace gearhip

using namespace gearhip;

extern "C" size_t gear_hip_search_workspace_bytes(int64_t num) { return search_ws_bytes(num); }

extern "C" int gear_hip_upper_bound_f64(const double *prefix, int64_t n, const float *u,
                                        int64_t num, int unit_uniforms, int64_t *idx_out,
                                        const float *priorities, double beta, float *weights_out,
                                        void *workspace, size_t workspace_bytes, void *stream) {
  if (n < 0 || num < 0) return GEAR_HIP_EINVAL;
  if (num == 0) return 0;
  if (n == 0 || !prefix || !u || !idx_out) return GEAR_HIP_EINVAL;
  if ((priorities == nullptr) != (weights_out == nullptr)) return GEAR_HIP_EINVAL;
  const int64_t blocks = ceil_div64(num, kSearchBlock);
  const int64_t nblocks = ceil_div64(num, kBlock);
  if (blocks >= 0x7fffffffll) return GEAR_HIP_ERANGE;
  double *wraw = nullptr, *bmax = nullptr;
  if (priorities) {
    if (!workspace || workspace_bytes < search_ws_bytes(num) ||
        (reinterpret_cast<uintptr_t>(workspace) & 7))
      return GEAR_HIP_EWORKSPACE;
    wraw = static_cast<double *>(workspace);
    bmax = reinterpret_cast<double *>(static_cast<char *>(workspace) +
                                      align_up((size_t)num * 8, 256));
  }
  hipStream_t st = as_stream(stream);
  search_f64_kernel<<<dim3((unsigned)blocks), dim3(kSearchBlock), 0, st>>>(
      prefix, n, u, num, unit_uniforms ? 1 : 0, idx_out, priorities, beta, wraw, bmax);
  GEARHIP_RETURN_IF_LAUNCH_FAILED();
  if (priorities) {
    normalise_kernel<<<dim3((unsigned)nblocks), dim3(kBlock), 0, st>>>(wraw, bmax, (int)blocks,
                                                                      num, weights_out);
    GEARHIP_RETURN_IF_LAUNCH_FAILED();
  }
  return 0;
}

extern "C" int gear_hip_upper_bound_i64(const int64_t *prefix, int64_t n, const void *u,
                                        int64_t num, int unit_uniforms, int64_t *idx_out,
                                        void *stream) {
  if (n < 0 || num < 0) return GEAR_HIP_EINVAL;
  if (num == 0) return 0;
  if (n == 0 || !prefix || !u || !idx_out) return GEAR_HIP_EINVAL;
  const int64_t blocks = ceil_div64(num, kSearchBlock);
  if (blocks >= 0x7fffffffll) return GEAR_HIP_ERANGE;
  search_i64_kernel<<<dim3((unsigned)blocks), dim3(kSearchBlock), 0, as_stream(stream)>>>(
      DrawI64{prefix, n, u, unit_uniforms ? 1 : 0}, num, idx_out);
  GEARHIP_RETURN_IF_LAUNCH_FAILED();
  return 0;
}

extern "C" size_t gear_hip_sample_workspace_bytes(int64_t num) { return sample_ws(num).total; }

extern "C" int gear_hip_sample_sorted_f64(const double *prefix, int64_t n, const float *u,
                                          int64_t num, int unit_uniforms, int64_t *sorted_out,
                                          int64_t trajectory_length, int64_t modulo,
                                          int64_t *idxs, int64_t *tss, int64_t *lens,
                                          void *workspace, size_t workspace_bytes, void *stream) {
  if (n < 0 || num < 0 || trajectory_length < 0 || modulo < 0) return GEAR_HIP_EINVAL;
  if (num == 0) return 0;
  if (n == 0 || !prefix || !u) return GEAR_HIP_EINVAL;
  if (trajectory_length > 0 && (!idxs || !tss)) return GEAR_HIP_EINVAL;
  if (trajectory_length == 0 && !sorted_out) return GEAR_HIP_EINVAL;
  int key_bits = 0;
  while (key_bits < 63 && ((uint64_t)(n - 1) >> key_bits) != 0) ++key_bits;
  hipStream_t st = as_stream(stream);
  const SampleWs w = sample_ws(num);
  if (!workspace || workspace_bytes < w.total || (reinterpret_cast<uintptr_t>(workspace) & 7))
    return GEAR_HIP_EWORKSPACE;
  char *ws = static_cast<char *>(workspace);
  int64_t *raw = reinterpret_cast<int64_t *>(ws + w.raw);
  const int64_t blocks = ceil_div64(num, kBlock);
  const int64_t sblocks = ceil_div64(num, kSearchBlock);
  if (sblocks >= 0x7fffffffll) return GEAR_HIP_ERANGE;
  const Split split{sorted_out, trajectory_length, modulo, idxs, tss, lens};
  search_f64_kernel<<<dim3((unsigned)sblocks), dim3(kSearchBlock), 0, st>>>(
      prefix, n, u, num, unit_uniforms ? 1 : 0, raw, nullptr, 0.0, nullptr, nullptr);
  GEARHIP_RETURN_IF_LAUNCH_FAILED();
  if (num <= radix::kRankMax && n < (1ll << 32)) {
    rank_split_kernel<<<dim3((unsigned)ceil_div64(num, kWave)), dim3(radix::kRankBlock), 0, st>>>(
        raw, (int)num, split);
    GEARHIP_RETURN_IF_LAUNCH_FAILED();
    return 0;
  }
  int64_t *sorted = sorted_out ? sorted_out : reinterpret_cast<int64_t *>(ws + w.sorted);
  int rc = radix::sort_pairs<uint64_t, uint64_t>(
      reinterpret_cast<const uint64_t *>(raw), reinterpret_cast<uint64_t *>(sorted), nullptr,
      nullptr, reinterpret_cast<uint64_t *>(ws + w.ktmp), nullptr, num, 0, key_bits,
      reinterpret_cast<uint32_t *>(ws + w.hist), st);
  if (rc) return rc;
  if (trajectory_length > 0) {
    split_sorted_kernel<<<dim3((unsigned)blocks), dim3(kBlock), 0, st>>>(
        sorted, num, trajectory_length, modulo, idxs, tss, lens);
    GEARHIP_RETURN_IF_LAUNCH_FAILED();
  }
  return 0;
}

namespace gearhip {
namespace {

int check_lookup(const Lookup &look) {
  if (look.index_n < 0 || look.lengths_n < 0) return GEAR_HIP_EINVAL;
  if ((look.lens || look.starts) && !look.lengths_table) return GEAR_HIP_EINVAL;
  if (look.starts && (!look.start_u || look.window < 1)) return GEAR_HIP_EINVAL;
  if (!look.sampled && !look.local && !look.lens && !look.starts) return GEAR_HIP_EINVAL;
  return 0;
}

// raw: num positions on the device (each in [0, bound)); sorted ascending, then looked up.
int sort_and_look_up(const int64_t *raw, int64_t num, int64_t bound, const Lookup &look, char *ws,
                     const SampleWs &w, hipStream_t st) {
  if (num <= radix::kRankMax && bound <= (1ll << 32)) {
    rank_lookup_kernel<<<dim3((unsigned)ceil_div64(num, kWave)), dim3(radix::kRankBlock), 0, st>>>(
        raw, (int)num, look);
    GEARHIP_RETURN_IF_LAUNCH_FAILED();
    return 0;
  }
  int key_bits = 1;
  while (key_bits < 63 && ((uint64_t)(bound - 1) >> key_bits) != 0) ++key_bits;
  int64_t *sorted = reinterpret_cast<int64_t *>(ws + w.sorted);
  const int rc = radix::sort_pairs<uint64_t, uint64_t>(
      reinterpret_cast<const uint64_t *>(raw), reinterpret_cast<uint64_t *>(sorted), nullptr,
      nullptr, reinterpret_cast<uint64_t *>(ws + w.ktmp), nullptr, num, 0, key_bits,
      reinterpret_cast<uint32_t *>(ws + w.hist), st);
  if (rc) return rc;
  lookup_kernel<<<dim3((unsigned)ceil_div64(num, kBlock)), dim3(kBlock), 0, st>>>(sorted, num, look);
  GEARHIP_RETURN_IF_LAUNCH_FAILED();
  return 0;
}

}  // namespace
}  // namespace gearhip

extern "C" int gear_hip_sample_lookup_f64(const double *prefix, int64_t n, const float *u,
                                          int64_t num, int unit_uniforms,
                                          const int64_t *index_table, int64_t index_offset,
                                          const int64_t *lengths_table, int64_t lengths_n,
                                          int64_t *sampled_out, int64_t *local_out,
                                          int64_t *lens_out, void *workspace,
                                          size_t workspace_bytes, void *stream) {
  if (n < 0 || num < 0) return GEAR_HIP_EINVAL;
  if (num == 0) return 0;
  if (n == 0 || !prefix || !u) return GEAR_HIP_EINVAL;
  const Lookup look{index_table, n, index_offset, lengths_table, lengths_n, sampled_out, local_out,
                    lens_out};
  int rc = check_lookup(look);
  if (rc) return rc;
  const SampleWs w = sample_ws(num);
  if (!workspace || workspace_bytes < w.total || (reinterpret_cast<uintptr_t>(workspace) & 7))
    return GEAR_HIP_EWORKSPACE;
  const int64_t sblocks = ceil_div64(num, kSearchBlock);
  if (sblocks >= 0x7fffffffll) return GEAR_HIP_ERANGE;
  char *ws = static_cast<char *>(workspace);
  int64_t *raw = reinterpret_cast<int64_t *>(ws + w.raw);
  hipStream_t st = as_stream(stream);
  search_f64_kernel<<<dim3((unsigned)sblocks), dim3(kSearchBlock), 0, st>>>(
      prefix, n, u, num, unit_uniforms ? 1 : 0, raw, nullptr, 0.0, nullptr, nullptr);
  GEARHIP_RETURN_IF_LAUNCH_FAILED();
  return sort_and_look_up(raw, num, n, look, ws, w, st);
}

extern "C" int gear_hip_sample_lookup_i64(const int64_t *prefix, int64_t n, const void *u,
                                          int64_t num, int unit_uniforms,
                                          const int64_t *index_table, int64_t index_offset,
                                          const int64_t *lengths_table, int64_t lengths_n,
                                          int64_t *sampled_out, int64_t *local_out,
                                          int64_t *lens_out, const double *start_uniforms,
                                          int64_t window, int64_t *starts_out, void *workspace,
                                          size_t workspace_bytes, void *stream) {
  if (n < 0 || num < 0) return GEAR_HIP_EINVAL;
  if (num == 0) return 0;
  if (n == 0 || !prefix || !u) return GEAR_HIP_EINVAL;
  Lookup look{index_table, n, index_offset, lengths_table, lengths_n, sampled_out, local_out,
              lens_out};
  look.start_u = start_uniforms;
  look.window = window;
  look.starts = starts_out;
  int rc = check_lookup(look);
  if (rc) return rc;
  const SampleWs w = sample_ws(num);
  if (!workspace || workspace_bytes < w.total || (reinterpret_cast<uintptr_t>(workspace) & 7))
    return GEAR_HIP_EWORKSPACE;
  const int64_t sblocks = ceil_div64(num, kSearchBlock);
  if (sblocks >= 0x7fffffffll) return GEAR_HIP_ERANGE;
  char *ws = static_cast<char *>(workspace);
  int64_t *raw = reinterpret_cast<int64_t *>(ws + w.raw);
  hipStream_t st = as_stream(stream);
  const DrawI64 draw{prefix, n, u, unit_uniforms ? 1 : 0};
  search_i64_kernel<<<dim3((unsigned)sblocks), dim3(kSearchBlock), 0, st>>>(draw, num, raw);
  GEARHIP_RETURN_IF_LAUNCH_FAILED();
  return sort_and_look_up(raw, num, n, look, ws, w, st);
}

extern "C" int gear_hip_sort_lookup_i64(const int64_t *positions, int64_t num, int64_t bound,
                                        const int64_t *index_table, int64_t index_n,
                                        int64_t index_offset, const int64_t *lengths_table,
                                        int64_t lengths_n, int64_t *sampled_out,
                                        int64_t *local_out, int64_t *lens_out, void *workspace,
                                        size_t workspace_bytes, void *stream) {
  if (num < 0 || bound <= 0) return GEAR_HIP_EINVAL;
  if (num == 0) return 0;
  if (!positions) return GEAR_HIP_EINVAL;
  const Lookup look{index_table, index_n, index_offset, lengths_table, lengths_n, sampled_out,
                    local_out, lens_out};
  int rc = check_lookup(look);
  if (rc) return rc;
  const SampleWs w = sample_ws(num);
  if (!workspace || workspace_bytes < w.total || (reinterpret_cast<uintptr_t>(workspace) & 7))
    return GEAR_HIP_EWORKSPACE;
  return sort_and_look_up(positions, num, bound, look, static_cast<char *>(workspace), w,
                          as_stream(stream));
}

extern "C" int gear_hip_lookup_i64(const int64_t *positions, int64_t num,
                                   const int64_t *index_table, int64_t index_n,
                                   int64_t index_offset, const int64_t *lengths_table,
                                   int64_t lengths_n, int64_t *sampled_out, int64_t *local_out,
                                   int64_t *lens_out, void *stream) {
  if (num < 0) return GEAR_HIP_EINVAL;
  if (num == 0) return 0;
  if (!positions) return GEAR_HIP_EINVAL;
  const Lookup look{index_table, index_n, index_offset, lengths_table, lengths_n, sampled_out,
                    local_out, lens_out};
  int rc = check_lookup(look);
  if (rc) return rc;
  const int64_t blocks = ceil_div64(num, kBlock);
  if (blocks >= 0x7fffffffll) return GEAR_HIP_ERANGE;
  lookup_kernel<<<dim3((unsigned)blocks), dim3(kBlock), 0, as_stream(stream)>>>(positions, num,
                                                                               look);
  GEARHIP_RETURN_IF_LAUNCH_FAILED();
  return 0;
}
