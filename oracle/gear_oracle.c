/*
 * gear_oracle.c — TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * A plain-C, single-threaded CPU restatement of the algorithms on GEAR's replay-sampling hot
 * path, written from the reference sources cited at each function (paths relative to the
 * bigrl-team/gear tree).  Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg
 * may load this library; nothing under gear_amd/ links, imports or calls it.
 *
 * Parity status of each function (what pins it, besides being read against the source):
 *   oracle_layout        closed form + tests/test_table.py:15-24 sizes            (pinned)
 *   oracle_sub           hand vector from tests/test_sub.py:10-28 + brute force   (pinned)
 *   oracle_subcopy       numpy fancy-index gather + examples/.../misc.py:16-29    (pinned)
 *   oracle_subcopy_mt    equality with oracle_subcopy                             (pinned)
 *   oracle_vcopy/copy    numpy slicing + tests/test_copy.py:5-28                  (pinned)
 *   oracle_scan_*        numpy.cumsum (fp64 / int64), integer-valued closed forms (pinned)
 *   oracle_sum_f32       math.fsum                                                (pinned)
 *   oracle_upper_bound_* numpy.searchsorted(side="right") + linear brute force    (pinned)
 *   oracle_is_weights    closed form evaluated with Python floats                 (pinned)
 *   oracle_topk_f32      numpy.argsort(-w, kind="stable")[:k]                     (pinned)
 *   oracle_sort_i64      numpy.argsort(kind="stable")                             (pinned)
 *   oracle_scatter_f32   Python loop "last write wins" (src/index/request.cc:41-51) (pinned)
 * The random streams of torch.randint / torch.multinomial inside the reference samplers
 * (gear/sampler/global_sampler.py:121-129,170) are properties of torch 1.13 and are NOT
 * restated here: "parity unpinned" at that boundary; draws are an input to this path.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORACLE_API __attribute__((visibility("default")))

/* ---- A1: table layout.  src/storage/table.cc:8-25, src/storage/specs.cc:10-14,25-29 -------- */
/* step_bytes[c] = ColumnSpec::size() (element size times the product of the shape).
 * accu[c] = sum of step_bytes[0..c) (accu_strides, table.cc:21-24), accu has ncols+1 entries.
 * trajectory_stride = T * sum(step_bytes) (table.cc:14-16); table bytes = stride * capacity
 * (table.cc:18).  Byte address of (trajectory i, column c, step t), from
 * src/storage/handler.cc:93-96,105-106,120 and :223-229:
 *     i * trajectory_stride + accu[c] * T + t * step_bytes[c]                                 */
ORACLE_API void oracle_layout(int64_t ncols, const int64_t *step_bytes, int64_t T,
                              int64_t capacity, int64_t *accu, int64_t *trajectory_stride,
                              int64_t *table_bytes) {
  int64_t sum = 0;
  accu[0] = 0;
  for (int64_t c = 0; c < ncols; ++c) {
    sum += step_bytes[c];
    accu[c + 1] = sum;
  }
  *trajectory_stride = sum * T;
  *table_bytes = sum * T * capacity;
}

/* ---- A3: CpuTrajectoryStorageHandler::sub.  src/storage/handler.cc:78-131 ------------------ */
ORACLE_API int64_t oracle_sub(int64_t num, const int64_t *idxs, const int64_t *tss,
                              const int64_t *lens, int pad_head, int64_t ofst, int64_t span,
                              int64_t traj_stride, int64_t step_bytes, int64_t col_base,
                              int64_t *src_offsets, int64_t *dst_offsets, int64_t *copy_lens) {
  const int64_t expected = span * step_bytes; /* handler.cc:98 */
  for (int64_t i = 0; i < num; ++i) {
    const int64_t base = idxs[i] * traj_stride + col_base; /* :105-106 */
    int64_t start = tss[i] + ofst;                          /* :107 */
    if (start < 0) start = 0;
    int64_t end = start + span; /* :108 */
    if (end > lens[i]) end = lens[i];
    start *= step_bytes; /* :110-111 */
    end *= step_bytes;
    int64_t n = end - start; /* :112 */
    if (n < 0) n = 0;
    int64_t d = pad_head ? expected - n : 0; /* :114-116 */
    d += expected * i;                        /* :117 */
    copy_lens[i] = n;
    src_offsets[i] = base + start;
    dst_offsets[i] = d;
  }
  return expected; /* :130 */
}

/* ---- A5: slice gathers.  src/cuda/copy.cu:12-89 (what the kernels compute, as memcpy) ------ */
ORACLE_API void oracle_vcopy(const uint8_t *src, uint8_t *dst, int64_t num,
                             const int64_t *src_offsets, const int64_t *dst_offsets,
                             const int64_t *strides) {
  for (int64_t g = 0; g < num; ++g)
    if (strides[g] > 0) memcpy(dst + dst_offsets[g], src + src_offsets[g], (size_t)strides[g]);
}

ORACLE_API void oracle_copy(const uint8_t *src, uint8_t *dst, int64_t num,
                            const int64_t *src_offsets, const int64_t *dst_offsets,
                            int64_t stride) {
  for (int64_t g = 0; g < num; ++g)
    if (stride > 0) memcpy(dst + dst_offsets[g], src + src_offsets[g], (size_t)stride);
}

/* ---- A4: fused window gather.  src/cuda/copy.cu:91-134 + src/storage/handler.cc:133-154 ---- */
/* Per window g (copy.cu:110-123): lsub=max(ts+ofst,0); rsub=min(lsub+span,len);
 * n=step_bytes*(rsub-lsub) (nothing copied when negative, :117); npad=(dst_stride-n)*pad_head;
 * from src + traj_stride*idx + col_base + lsub*step_bytes to dst + dst_stride*g + npad.
 * zero_fill reproduces the torch.zeros the caller applies first
 * (gear/loader/offline_loader.py:181-189).  mask (may be NULL): uint8[num, span].            */
ORACLE_API void oracle_subcopy(const uint8_t *src, uint8_t *dst, int64_t num,
                               const int64_t *idxs, const int64_t *tss, const int64_t *lens,
                               int pad_head, int64_t ofst, int64_t span, int64_t traj_stride,
                               int64_t step_bytes, int64_t col_base, int64_t dst_stride,
                               int zero_fill, uint8_t *mask) {
  for (int64_t g = 0; g < num; ++g) {
    int64_t lsub = tss[g] + ofst;
    if (lsub < 0) lsub = 0;
    int64_t rsub = lsub + span;
    if (rsub > lens[g]) rsub = lens[g];
    int64_t steps = rsub - lsub;
    if (steps < 0) steps = 0;
    const int64_t n = steps * step_bytes;
    const int64_t npad = pad_head ? dst_stride - n : 0;
    uint8_t *w = dst + dst_stride * g;
    if (zero_fill) memset(w, 0, (size_t)dst_stride);
    if (n > 0)
      memcpy(w + npad, src + traj_stride * idxs[g] + col_base + lsub * step_bytes, (size_t)n);
    if (mask) {
      for (int64_t j = 0; j < span; ++j)
        mask[g * span + j] = pad_head ? (uint8_t)(j >= span - steps) : (uint8_t)(j < steps);
    }
  }
}

/* The same gather with the windows split over `threads` host threads (windows are independent
 * units; each thread runs oracle_subcopy on a contiguous share).  Only the all-cores leg of the
 * CPU baseline uses it; results are identical to oracle_subcopy by construction (tested).    */
ORACLE_API void oracle_subcopy_mt(const uint8_t *src, uint8_t *dst, int64_t num,
                                  const int64_t *idxs, const int64_t *tss, const int64_t *lens,
                                  int pad_head, int64_t ofst, int64_t span, int64_t traj_stride,
                                  int64_t step_bytes, int64_t col_base, int64_t dst_stride,
                                  int zero_fill, uint8_t *mask, int threads) {
  if (threads < 1) threads = 1;
#pragma omp parallel for num_threads(threads) schedule(static)
  for (int t = 0; t < threads; ++t) {
    const int64_t lo = num * t / threads, hi = num * (t + 1) / threads;
    if (hi > lo)
      oracle_subcopy(src, dst + dst_stride * lo, hi - lo, idxs + lo, tss + lo, lens + lo, pad_head,
                     ofst, span, traj_stride, step_bytes, col_base, dst_stride, zero_fill,
                     mask ? mask + lo * span : NULL);
  }
}

/* ---- A6: prefix sum.  Intent of src/cuda/one_dim_prefix_sum.cu:125-234 (inclusive scan of the
 * priorities), accumulated sequentially in fp64 as the benchmark's "fp64 prefix sum" asks ---------- */
ORACLE_API void oracle_scan_f32_f64(const float *in, double *out, int64_t n) {
  double acc = 0.0;
  for (int64_t i = 0; i < n; ++i) {
    acc += (double)in[i];
    out[i] = acc;
  }
}

ORACLE_API void oracle_scan_i64(const int64_t *in, int64_t *out, int64_t n) {
  int64_t acc = 0;
  for (int64_t i = 0; i < n; ++i) {
    acc += in[i];
    out[i] = acc;
  }
}

/* The same prefix sum over `threads` host threads: every thread sums a contiguous chunk, the
 * chunk sums are scanned sequentially, every thread then scans its chunk from its offset.  Only
 * the all-cores leg of the CPU baseline uses it.  The summation order differs from the
 * sequential scan's, so results agree to rounding (exactly on integer-valued input; tested). */
ORACLE_API void oracle_scan_f32_f64_mt(const float *in, double *out, int64_t n, int threads) {
  if (threads < 1) threads = 1;
  if (threads > 256) threads = 256;
  double sums[256];
#pragma omp parallel for num_threads(threads) schedule(static)
  for (int t = 0; t < threads; ++t) {
    const int64_t lo = n * t / threads, hi = n * (t + 1) / threads;
    double acc = 0.0;
    for (int64_t i = lo; i < hi; ++i) acc += (double)in[i];
    sums[t] = acc;
  }
  double run = 0.0;
  for (int t = 0; t < threads; ++t) {
    const double s = sums[t];
    sums[t] = run;
    run += s;
  }
#pragma omp parallel for num_threads(threads) schedule(static)
  for (int t = 0; t < threads; ++t) {
    const int64_t lo = n * t / threads, hi = n * (t + 1) / threads;
    double acc = sums[t];
    for (int64_t i = lo; i < hi; ++i) {
      acc += (double)in[i];
      out[i] = acc;
    }
  }
}

/* Sum of fp32 values (src/cuda/one_dim_sum.cu:22-74 computes it with fp32 atomics); here the
 * sequential fp64 sum, rounded once to fp32. */
ORACLE_API double oracle_sum_f32(const float *in, int64_t n) {
  double acc = 0.0;
  for (int64_t i = 0; i < n; ++i) acc += (double)in[i];
  return acc;
}

/* ---- A6: search.  idx = min(#{i : prefix[i] <= t}, n-1), i.e. std::upper_bound -------------- */
static int64_t upper_bound_f64(const double *p, int64_t n, double t) {
  int64_t lo = 0, hi = n; /* first index with p[i] > t */
  while (lo < hi) {
    const int64_t mid = lo + ((hi - lo) >> 1);
    if (p[mid] <= t)
      lo = mid + 1;
    else
      hi = mid;
  }
  return lo;
}

ORACLE_API void oracle_upper_bound_f64(const double *prefix, int64_t n, const float *u,
                                       int64_t num, int unit_uniforms, int64_t *idx_out) {
  if (n <= 0) return;
  const double total = prefix[n - 1];
  for (int64_t j = 0; j < num; ++j) {
    const double t = unit_uniforms ? (double)u[j] * total : (double)u[j];
    int64_t i = upper_bound_f64(prefix, n, t);
    if (i > n - 1) i = n - 1;
    idx_out[j] = i;
  }
}

/* The same search with the draws split over `threads` host threads (identical results). */
ORACLE_API void oracle_upper_bound_f64_mt(const double *prefix, int64_t n, const float *u,
                                          int64_t num, int unit_uniforms, int64_t *idx_out,
                                          int threads) {
  if (threads < 1) threads = 1;
#pragma omp parallel for num_threads(threads) schedule(static)
  for (int t = 0; t < threads; ++t) {
    const int64_t lo = num * t / threads, hi = num * (t + 1) / threads;
    if (hi > lo) oracle_upper_bound_f64(prefix, n, u + lo, hi - lo, unit_uniforms, idx_out + lo);
  }
}

ORACLE_API void oracle_upper_bound_i64(const int64_t *prefix, int64_t n, const void *u,
                                       int64_t num, int unit_uniforms, int64_t *idx_out) {
  if (n <= 0) return;
  const int64_t total = prefix[n - 1];
  for (int64_t j = 0; j < num; ++j) {
    int64_t t;
    if (unit_uniforms)
      t = (int64_t)floor(((const double *)u)[j] * (double)total);
    else
      t = ((const int64_t *)u)[j];
    int64_t lo = 0, hi = n;
    while (lo < hi) {
      const int64_t mid = lo + ((hi - lo) >> 1);
      if (prefix[mid] <= t)
        lo = mid + 1;
      else
        hi = mid;
    }
    if (lo > n - 1) lo = n - 1;
    idx_out[j] = lo;
  }
}

/* Importance weights of benchmark config 2: w_j = (n * p[idx_j] / total)^(-beta) in fp64,
 * divided by the maximum over the batch, stored as fp32.  Not in the reference. */
ORACLE_API void oracle_is_weights(const float *priorities, int64_t n, double total,
                                  const int64_t *idx, int64_t num, double beta, float *out) {
  double wmax = 0.0;
  double *w = (double *)malloc(sizeof(double) * (size_t)(num > 0 ? num : 1));
  for (int64_t j = 0; j < num; ++j) {
    w[j] = pow((double)n * (double)priorities[idx[j]] / total, -beta);
    if (w[j] > wmax) wmax = w[j];
  }
  for (int64_t j = 0; j < num; ++j) out[j] = (float)(w[j] / wmax);
  free(w);
}

/* ---- A6: top-k.  Semantics of torch.topk(weights, k, largest=True) as used by TopKSampler
 * (gear/sampler/global_sampler.py:195-199); ties: smaller index first (stable descending). ---- */
typedef struct {
  float v;
  int64_t i;
} oracle_vi;

static int cmp_desc_stable(const void *a, const void *b) {
  const oracle_vi *x = (const oracle_vi *)a, *y = (const oracle_vi *)b;
  if (x->v > y->v) return -1;
  if (x->v < y->v) return 1;
  return (x->i > y->i) - (x->i < y->i);
}

static int cmp_i64(const void *a, const void *b) {
  const int64_t x = *(const int64_t *)a, y = *(const int64_t *)b;
  return (x > y) - (x < y);
}

/* Keeps a k-sized candidate set by quickselect on (value desc, index asc), then orders it. */
/* a[0, k) becomes the k first elements of the total order (value descending, index ascending),
 * sorted: quickselect with a seeded pivot sequence, then qsort of the front. */
static void select_front(oracle_vi *a, int64_t n, int64_t k) {
  int64_t lo = 0, hi = n - 1;
  uint64_t rng = 0x9E3779B97F4A7C15ull;
  while (lo < hi) {
    rng ^= rng << 13;
    rng ^= rng >> 7;
    rng ^= rng << 17;
    const int64_t pi = lo + (int64_t)(rng % (uint64_t)(hi - lo + 1));
    const oracle_vi pv = a[pi];
    int64_t i = lo, j = hi;
    while (i <= j) {
      while (cmp_desc_stable(&a[i], &pv) < 0) ++i;
      while (cmp_desc_stable(&a[j], &pv) > 0) --j;
      if (i <= j) {
        const oracle_vi t = a[i];
        a[i] = a[j];
        a[j] = t;
        ++i;
        --j;
      }
    }
    if (k - 1 <= j)
      hi = j;
    else if (k - 1 >= i)
      lo = i;
    else
      break;
  }
  qsort(a, (size_t)k, sizeof(oracle_vi), cmp_desc_stable);
}

static void topk_emit(const float *w, const oracle_vi *a, int64_t k, int sorted_by_value,
                      float *values_out, int64_t *indices_out) {
  if (sorted_by_value) {
    for (int64_t j = 0; j < k; ++j) {
      if (values_out) values_out[j] = a[j].v;
      indices_out[j] = a[j].i;
    }
  } else {
    for (int64_t j = 0; j < k; ++j) indices_out[j] = a[j].i;
    qsort(indices_out, (size_t)k, sizeof(int64_t), cmp_i64);
    if (values_out)
      for (int64_t j = 0; j < k; ++j) values_out[j] = w[indices_out[j]];
  }
}

ORACLE_API void oracle_topk_f32(const float *w, int64_t n, int64_t k, int sorted_by_value,
                                float *values_out, int64_t *indices_out) {
  if (k <= 0 || n <= 0) return;
  if (k > n) k = n;
  oracle_vi *a = (oracle_vi *)malloc(sizeof(oracle_vi) * (size_t)n);
  for (int64_t i = 0; i < n; ++i) {
    a[i].v = w[i];
    a[i].i = i;
  }
  select_front(a, n, k);
  topk_emit(w, a, k, sorted_by_value, values_out, indices_out);
  free(a);
}

/* The same selection over `threads` host threads: every thread selects the top min(k, chunk)
 * of a contiguous chunk, the survivors (at most threads * k) go through one more selection.
 * Only the all-cores leg of the CPU baseline uses it; the result is identical to
 * oracle_topk_f32 (the total order is the same; tested). */
ORACLE_API void oracle_topk_f32_mt(const float *w, int64_t n, int64_t k, int sorted_by_value,
                                   float *values_out, int64_t *indices_out, int threads) {
  if (k <= 0 || n <= 0) return;
  if (k > n) k = n;
  if (threads < 1) threads = 1;
  if (threads > 256) threads = 256;
  oracle_vi *a = (oracle_vi *)malloc(sizeof(oracle_vi) * (size_t)n);
  int64_t kept[256];
#pragma omp parallel for num_threads(threads) schedule(static)
  for (int t = 0; t < threads; ++t) {
    const int64_t lo = n * t / threads, hi = n * (t + 1) / threads;
    for (int64_t i = lo; i < hi; ++i) {
      a[i].v = w[i];
      a[i].i = i;
    }
    const int64_t kk = k < hi - lo ? k : hi - lo;
    if (kk > 0) select_front(a + lo, hi - lo, kk);
    kept[t] = kk;
  }
  int64_t m = 0;
  for (int t = 0; t < threads; ++t) {
    const int64_t lo = n * t / threads;
    if (lo != m) memmove(a + m, a + lo, sizeof(oracle_vi) * (size_t)kept[t]);
    m += kept[t];
  }
  select_front(a, m, k);
  topk_emit(w, a, k, sorted_by_value, values_out, indices_out);
  free(a);
}

typedef struct {
  int64_t k;
  int64_t pos;
  int64_t v;
} oracle_kv;

static int cmp_kv(const void *a, const void *b) {
  const oracle_kv *x = (const oracle_kv *)a, *y = (const oracle_kv *)b;
  if (x->k != y->k) return (x->k > y->k) - (x->k < y->k);
  return (x->pos > y->pos) - (x->pos < y->pos);
}

ORACLE_API void oracle_sort_i64(const int64_t *keys_in, int64_t *keys_out, const int64_t *vals_in,
                                int64_t *vals_out, int64_t num) {
  oracle_kv *a = (oracle_kv *)malloc(sizeof(oracle_kv) * (size_t)(num > 0 ? num : 1));
  for (int64_t i = 0; i < num; ++i) {
    a[i].k = keys_in[i];
    a[i].pos = i;
    a[i].v = vals_in ? vals_in[i] : 0;
  }
  qsort(a, (size_t)num, sizeof(oracle_kv), cmp_kv);
  for (int64_t i = 0; i < num; ++i) {
    keys_out[i] = a[i].k;
    if (vals_out) vals_out[i] = a[i].v;
  }
  free(a);
}

/* ---- A7: priority update.  Indexset::set_weight per element (include/index/set.h:245-247);
 * duplicates: the later write stays (src/index/request.cc:41-51).  Out-of-range ignored. ------ */
ORACLE_API void oracle_scatter_f32(float *weights, int64_t n, const int64_t *idx,
                                   const float *values, int64_t num) {
  for (int64_t j = 0; j < num; ++j)
    if (idx[j] >= 0 && idx[j] < n) weights[idx[j]] = values[j];
}
