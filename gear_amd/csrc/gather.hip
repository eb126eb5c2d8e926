// Trajectory-window gather for gfx950: one kernel body shared by subcopy (window arithmetic fused
// on the device), vcopy/copy (explicit offsets) and the multi-column launch.
//
// Work decomposition.  A "slice" is one window of one column: a destination region
// [rp, rp+rl) of which [cs, cs+n) is copied from the table and the rest (padding) is zero.
// The destination is cut into 16-byte vectors on ABSOLUTE 16-byte boundaries, so every store in
// the hot loop is an aligned global_store_dwordx4; the matching source bytes are fetched with one
// global_load_dwordx4 at whatever byte alignment the table layout gives (the table has no
// padding: a window of fp32[17] steps starts on a 4-byte boundary, a uint8 column on any byte).
// Vectors that straddle the region edge or the copy/padding edge (at most four per slice) take a
// byte path.  A group of `tg` threads (power of two, 1..128) owns one chunk of tg*U consecutive
// vectors; lanes of a group take consecutive vectors so a wave reads and writes 1 KiB runs and a
// 128-thread workgroup covers one contiguous 4 KiB piece of a large window (source cache lines
// shared by neighbouring pieces are then fetched twice only at 4 KiB boundaries).
// Each thread issues its U loads before its first store to keep U*16 bytes per lane in flight.
#include "common.hpp"

namespace gearhip {
namespace {

constexpr int kBlock = 128;       // threads per workgroup
constexpr int kMaxGroupShift = 7;  // a group never spans workgroups: at most 128 threads

enum GatherMode { kSubcopy = 0, kVcopy = 1, kCopy = 2 };

// vector u of a lane: lanes of a group take consecutive vectors (coalesced 1 KiB per wave)
#define GEARHIP_VEC_INDEX(k0, u, tg, lane, U) ((k0) + (int64_t)(u) * (tg) + (lane))

struct ColumnArgs {
  uint8_t *dst;
  uint8_t *mask;
  int64_t ofst, span, step_bytes, col_base, dst_stride;
  int64_t cps;          // chunks per slice
  int64_t block_begin;  // first block of this column in a multi-column grid
  int32_t pad_head, zero_fill;
  int32_t tg_shift;     // log2(threads per group)
  int32_t pad_;
};

struct GatherArgs {
  const uint8_t *src;
  int64_t num;
  const int64_t *a;  // subcopy: idxs        vcopy/copy: src_offsets
  const int64_t *b;  // subcopy: tss         vcopy/copy: dst_offsets
  const int64_t *c;  // subcopy: lens        vcopy: strides
  int64_t traj_stride;
  int64_t fixed_stride;  // copy mode
  int64_t capacity;      // subcopy: trajectories in the table, 0 = indices are not checked
  int64_t traj_len;      // subcopy: steps per trajectory, 0 = lengths are not clamped
};

struct MultiArgs {
  ColumnArgs col[GEAR_HIP_MAX_COLUMNS];
  int32_t ncols;
};

struct Slice {
  const uint8_t *sp;  // source of the first copied byte
  uint8_t *rp;        // first byte of the destination region
  int64_t rl;         // region length
  int64_t cs;         // copy range start, relative to rp
  int64_t n;          // copied bytes
};

// NT is a bit mask: 1 = non-temporal loads, 2 = non-temporal stores
template <int NT>
__device__ __forceinline__ u32x4 load16(const uint8_t *p) {
  if (NT & 1) return __builtin_nontemporal_load(reinterpret_cast<const u32x4_a1 *>(p));
  return reinterpret_cast<const u32x4_any *>(p)->v;
}

template <int NT>
__device__ __forceinline__ void store16(uint8_t *p, u32x4 v) {
  if (NT & 2)
    __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(p));
  else
    *reinterpret_cast<u32x4 *>(p) = v;
}

// Copies the part of slice `s` that belongs to group-chunk `c` (and c+cps, ... if the slice is
// longer than the launch was sized for).
template <int U, int NT>
__device__ __forceinline__ void gather_chunks(const Slice &s, int64_t c, int64_t cps, int lane,
                                              int tg) {
  const uintptr_t r0 = reinterpret_cast<uintptr_t>(s.rp);
  const int64_t head = (int64_t)(r0 & 15);
  uint8_t *ap = s.rp - head;  // 16-byte aligned
  const int64_t nvec = (head + s.rl + 15) >> 4;
  const int64_t ce = s.cs + s.n;
  const int64_t chunk = (int64_t)tg * U;

  for (int64_t k0 = c * chunk; k0 < nvec; k0 += cps * chunk) {
    u32x4 v[U];
    int kind[U];  // 0 nothing, 1 full aligned store, 2 byte path
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t k = GEARHIP_VEC_INDEX(k0, u, tg, lane, U);
      const int64_t lo = (k << 4) - head;
      const int64_t hi = lo + 16;
      kind[u] = 0;
      v[u] = u32x4{0u, 0u, 0u, 0u};
      if (k < nvec) {
        if (lo >= 0 && hi <= s.rl) {
          if (lo >= s.cs && hi <= ce) {
            v[u] = load16<NT>(s.sp + (lo - s.cs));
            kind[u] = 1;
          } else if (hi <= s.cs || lo >= ce) {
            kind[u] = 1;  // all padding
          } else {
            kind[u] = 2;
          }
        } else {
          kind[u] = 2;
        }
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int64_t k = GEARHIP_VEC_INDEX(k0, u, tg, lane, U);
      if (kind[u] == 1) store16<NT>(ap + (k << 4), v[u]);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (kind[u] == 2) {
        const int64_t k = GEARHIP_VEC_INDEX(k0, u, tg, lane, U);
        const int64_t lo = (k << 4) - head;
        for (int j = 0; j < 16; ++j) {
          const int64_t off = lo + j;
          if (off >= 0 && off < s.rl) {
            uint8_t b = 0;
            if (off >= s.cs && off < ce) b = s.sp[off - s.cs];
            s.rp[off] = b;
          }
        }
      }
    }
  }
}

// Window arithmetic of fused_subcopy_collect (src/cuda/copy.cu:110-123) in int64.
__device__ __forceinline__ Slice resolve_window(const GatherArgs &p, const ColumnArgs &col,
                                                int64_t g, int64_t *valid_steps) {
  const int64_t idx = p.a[g], ts = p.b[g];
  int64_t len = p.c[g];
  if (p.traj_len > 0 && len > p.traj_len) len = p.traj_len;
  if (p.capacity > 0 && (idx < 0 || idx >= p.capacity)) len = 0;  // nothing to read: all padding
  int64_t lsub = ts + col.ofst;
  if (lsub < 0) lsub = 0;
  int64_t rsub = lsub + col.span;
  if (rsub > len) rsub = len;
  int64_t steps = rsub - lsub;
  if (steps < 0) steps = 0;
  *valid_steps = steps;
  const int64_t n = steps * col.step_bytes;
  const int64_t npad = col.pad_head ? col.dst_stride - n : 0;
  Slice s;
  s.sp = p.src + idx * p.traj_stride + col.col_base + lsub * col.step_bytes;
  uint8_t *w0 = col.dst + g * col.dst_stride;
  if (col.zero_fill) {
    s.rp = w0;
    s.rl = col.dst_stride;
    s.cs = npad;
  } else {
    s.rp = w0 + npad;
    s.rl = n;
    s.cs = 0;
  }
  s.n = n;
  return s;
}

template <int U, int NT>
__device__ __forceinline__ void subcopy_body(const GatherArgs &p, const ColumnArgs &col,
                                             int64_t block) {
  const int64_t t = block * kBlock + threadIdx.x;
  const int64_t gid = t >> col.tg_shift;
  const int tg = 1 << col.tg_shift;
  const int lane = (int)(t & (tg - 1));
  int64_t g, c;
  if (col.cps == 1) {
    g = gid;
    c = 0;
  } else if (gid < 0x7fffffff) {
    g = (uint32_t)gid / (uint32_t)col.cps;
    c = gid - g * col.cps;
  } else {
    g = gid / col.cps;
    c = gid - g * col.cps;
  }
  if (g >= p.num) return;
  int64_t steps;
  const Slice s = resolve_window(p, col, g, &steps);
  if (col.mask != nullptr && c == 0) {
    uint8_t *m = col.mask + g * col.span;
    for (int64_t j = lane; j < col.span; j += tg)
      m[j] = col.pad_head ? (uint8_t)(j >= col.span - steps) : (uint8_t)(j < steps);
  }
  gather_chunks<U, NT>(s, c, col.cps, lane, tg);
}

template <int U, int NT>
__global__ __launch_bounds__(kBlock) void subcopy_kernel(GatherArgs p, ColumnArgs col) {
  subcopy_body<U, NT>(p, col, blockIdx.x);
}

template <int U, int NT>
__global__ __launch_bounds__(kBlock) void subcopy_multi_kernel(GatherArgs p, MultiArgs m) {
  // columns are laid out one after another along the grid; find this block's column
  int ci = 0;
  const int64_t b = blockIdx.x;
#pragma unroll 1
  for (int i = 1; i < m.ncols; ++i)
    if (b >= m.col[i].block_begin) ci = i;
  subcopy_body<U, NT>(p, m.col[ci], b - m.col[ci].block_begin);
}

template <int MODE, int U, int NT>
__global__ __launch_bounds__(kBlock) void slices_kernel(GatherArgs p, uint8_t *dst, int64_t cps,
                                                        int tg_shift) {
  const int64_t t = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  const int64_t gid = t >> tg_shift;
  const int tg = 1 << tg_shift;
  const int lane = (int)(t & (tg - 1));
  int64_t g, c;
  if (cps == 1) {
    g = gid;
    c = 0;
  } else {
    g = gid / cps;
    c = gid - g * cps;
  }
  if (g >= p.num) return;
  Slice s;
  s.n = (MODE == kCopy) ? p.fixed_stride : p.c[g];
  if (s.n < 0) s.n = 0;
  s.sp = p.src + p.a[g];
  s.rp = dst + p.b[g];
  s.rl = s.n;
  s.cs = 0;
  gather_chunks<U, NT>(s, c, cps, lane, tg);
}

// Device restatement of CpuTrajectoryStorageHandler::sub (src/storage/handler.cc:100-121).
__global__ __launch_bounds__(kBlock) void sub_kernel(int64_t num, const int64_t *idxs,
                                                     const int64_t *tss, const int64_t *lens,
                                                     int pad_head, int64_t ofst, int64_t span,
                                                     int64_t traj_stride, int64_t step_bytes,
                                                     int64_t col_base, int64_t *src_offsets,
                                                     int64_t *dst_offsets, int64_t *copy_lens) {
  const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (i >= num) return;
  const int64_t expected = span * step_bytes;
  int64_t start = tss[i] + ofst;
  if (start < 0) start = 0;
  int64_t end = start + span;
  if (end > lens[i]) end = lens[i];
  start *= step_bytes;
  end *= step_bytes;
  int64_t copy_len = end - start;
  if (copy_len < 0) copy_len = 0;
  copy_lens[i] = copy_len;
  src_offsets[i] = idxs[i] * traj_stride + col_base + start;
  dst_offsets[i] = expected * i + (pad_head ? expected - copy_len : 0);
}

// flat step index -> (trajectory, timestep, length = timestep + 1)
__global__ __launch_bounds__(kBlock) void split_kernel(const int64_t *__restrict__ flat,
                                                       int64_t num, int64_t T, int64_t modulo,
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

// out[j] = table[idx[j]] for 8-byte elements (timesteps / global indices of the sampled batch)
__global__ __launch_bounds__(kBlock) void take_kernel(const int64_t *__restrict__ table, int64_t n,
                                                      const int64_t *__restrict__ idx, int64_t num,
                                                      int64_t add, int64_t *__restrict__ out) {
  const int64_t j = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (j >= num) return;
  const int64_t i = idx[j];
  out[j] = (i >= 0 && i < n) ? table[i] + add : 0;
}

struct Shape {
  int tg_shift;
  int64_t cps;
  int64_t blocks;
};

// Threads per group and chunks per slice for slices of at most `max_region` destination bytes.
Shape plan(int64_t num, int64_t max_region, int U) {
  Shape s;
  int64_t nvec = (max_region + 30) >> 4;  // worst-case head misalignment of 15 bytes
  if (nvec < 1) nvec = 1;
  int64_t want = ceil_div64(nvec, U);
  int sh = 0;
  while ((1ll << sh) < want && sh < kMaxGroupShift) ++sh;
  s.tg_shift = sh;
  s.cps = ceil_div64(nvec, (int64_t)U << sh);
  const int64_t threads = num * s.cps * (1ll << sh);
  s.blocks = ceil_div64(threads, kBlock);
  return s;
}

// The one instantiation that is built: two vectors per thread (8 KiB per workgroup, many small
// workgroups) with non-temporal stores.  Measured on MI355X at the 2048 x 847 KB window shape
// that moves 6.1-6.3 TB/s; four or eight vectors per thread, or plain stores, stay between 5.1
// and 5.7 TB/s, non-temporal loads change nothing.
constexpr int kUnroll = 2;
constexpr int kNt = 2;  // bit mask: 1 = non-temporal loads, 2 = non-temporal stores

int fill_column(const gear_hip_column_desc &d, int64_t num, int U, ColumnArgs *out,
                int64_t *blocks) {
  if (d.dst == nullptr || d.span < 0 || d.step_bytes <= 0 || d.dst_stride < 0 || d.col_base < 0)
    return GEAR_HIP_EINVAL;
  if (d.span * d.step_bytes > d.dst_stride) return GEAR_HIP_EINVAL;
  if (reinterpret_cast<uintptr_t>(d.dst) & 15) return GEAR_HIP_EALIGN;
  const int64_t max_region = d.zero_fill ? d.dst_stride : d.span * d.step_bytes;
  const Shape s = plan(num, max_region, U);
  out->dst = static_cast<uint8_t *>(d.dst);
  out->mask = d.mask_out;
  out->ofst = d.ofst;
  out->span = d.span;
  out->step_bytes = d.step_bytes;
  out->col_base = d.col_base;
  out->dst_stride = d.dst_stride;
  out->cps = s.cps;
  out->block_begin = 0;
  out->pad_head = d.pad_head ? 1 : 0;
  out->zero_fill = d.zero_fill ? 1 : 0;
  out->tg_shift = s.tg_shift;
  out->pad_ = 0;
  *blocks = s.blocks;
  return 0;
}

int launch_subcopy(const GatherArgs &p, const ColumnArgs &col, int64_t blocks, hipStream_t st) {
  subcopy_kernel<kUnroll, kNt><<<dim3((unsigned)blocks), dim3(kBlock), 0, st>>>(p, col);
  GEARHIP_RETURN_IF_LAUNCH_FAILED();
  return 0;
}

int launch_multi(const GatherArgs &p, const MultiArgs &m, int64_t blocks, hipStream_t st) {
  subcopy_multi_kernel<kUnroll, kNt><<<dim3((unsigned)blocks), dim3(kBlock), 0, st>>>(p, m);
  GEARHIP_RETURN_IF_LAUNCH_FAILED();
  return 0;
}

template <int MODE>
int launch_slices(const GatherArgs &p, uint8_t *dst, int64_t max_len, hipStream_t st) {
  const Shape s = plan(p.num, max_len, kUnroll);
  if (s.blocks >= 0x7fffffffll) return GEAR_HIP_ERANGE;
  slices_kernel<MODE, kUnroll, kNt><<<dim3((unsigned)s.blocks), dim3(kBlock), 0, st>>>(
      p, dst, s.cps, s.tg_shift);
  GEARHIP_RETURN_IF_LAUNCH_FAILED();
  return 0;
}

}  // namespace
}  // namespace gearhip

using namespace gearhip;

extern "C" int gear_hip_subcopy(const void *src, void *dst, int64_t num, const int64_t *idxs,
                                const int64_t *tss, const int64_t *lens, int pad_head,
                                int64_t ofst, int64_t span, int64_t traj_stride,
                                int64_t step_bytes, int64_t col_base, int64_t dst_stride,
                                int zero_fill, uint8_t *mask_out, void *stream) {
  if (num < 0) return GEAR_HIP_EINVAL;
  if (num == 0) return 0;
  if (!src || !idxs || !tss || !lens || traj_stride < 0) return GEAR_HIP_EINVAL;
  gear_hip_column_desc d;
  d.dst = dst;
  d.mask_out = mask_out;
  d.ofst = ofst;
  d.span = span;
  d.step_bytes = step_bytes;
  d.col_base = col_base;
  d.dst_stride = dst_stride;
  d.pad_head = pad_head;
  d.zero_fill = zero_fill;
  const int U = kUnroll;
  ColumnArgs col;
  int64_t blocks = 0;
  int rc = fill_column(d, num, U, &col, &blocks);
  if (rc) return rc;
  if (blocks >= 0x7fffffffll) return GEAR_HIP_ERANGE;
  GatherArgs p{static_cast<const uint8_t *>(src), num, idxs, tss, lens, traj_stride, 0, 0, 0};
  return launch_subcopy(p, col, blocks, as_stream(stream));
}

extern "C" int gear_hip_subcopy_multi(const void *src, int64_t num, const int64_t *idxs,
                                      const int64_t *tss, const int64_t *lens,
                                      int64_t traj_stride, const gear_hip_column_desc *cols,
                                      int ncols, void *stream) {
  return gear_hip_subcopy_multi_checked(src, num, idxs, tss, lens, traj_stride, 0, 0, cols, ncols,
                                        stream);
}

extern "C" int gear_hip_subcopy_multi_checked(const void *src, int64_t num, const int64_t *idxs,
                                              const int64_t *tss, const int64_t *lens,
                                              int64_t traj_stride, int64_t capacity,
                                              int64_t trajectory_length,
                                              const gear_hip_column_desc *cols, int ncols,
                                              void *stream) {
  if (num < 0 || ncols < 0 || ncols > GEAR_HIP_MAX_COLUMNS || capacity < 0 || trajectory_length < 0)
    return GEAR_HIP_EINVAL;
  if (num == 0 || ncols == 0) return 0;
  if (!src || !idxs || !tss || !lens || !cols || traj_stride < 0) return GEAR_HIP_EINVAL;
  const int U = kUnroll;
  MultiArgs m;
  m.ncols = ncols;
  int64_t total = 0;
  for (int i = 0; i < ncols; ++i) {
    int64_t blocks = 0;
    int rc = fill_column(cols[i], num, U, &m.col[i], &blocks);
    if (rc) return rc;
    m.col[i].block_begin = total;
    total += blocks;
  }
  for (int i = ncols; i < GEAR_HIP_MAX_COLUMNS; ++i) m.col[i] = m.col[0];
  if (total >= 0x7fffffffll) return GEAR_HIP_ERANGE;
  GatherArgs p{static_cast<const uint8_t *>(src), num,        idxs, tss, lens, traj_stride, 0,
               capacity,                          trajectory_length};
  return launch_multi(p, m, total, as_stream(stream));
}

extern "C" int gear_hip_vcopy(const void *src, void *dst, int64_t num,
                              const int64_t *src_offsets, const int64_t *dst_offsets,
                              const int64_t *strides, int64_t max_stride, void *stream) {
  if (num < 0 || max_stride < 0) return GEAR_HIP_EINVAL;
  if (num == 0) return 0;
  if (!src || !dst || !src_offsets || !dst_offsets || !strides) return GEAR_HIP_EINVAL;
  GatherArgs p{static_cast<const uint8_t *>(src), num, src_offsets, dst_offsets, strides, 0, 0, 0, 0};
  return launch_slices<kVcopy>(p, static_cast<uint8_t *>(dst), max_stride, as_stream(stream));
}

extern "C" int gear_hip_copy(const void *src, void *dst, int64_t num, const int64_t *src_offsets,
                             const int64_t *dst_offsets, int64_t stride, void *stream) {
  if (num < 0 || stride < 0) return GEAR_HIP_EINVAL;
  if (num == 0 || stride == 0) return 0;
  if (!src || !dst || !src_offsets || !dst_offsets) return GEAR_HIP_EINVAL;
  GatherArgs p{static_cast<const uint8_t *>(src), num, src_offsets, dst_offsets, nullptr, 0,
               stride, 0, 0};
  return launch_slices<kCopy>(p, static_cast<uint8_t *>(dst), stride, as_stream(stream));
}

extern "C" int gear_hip_sub(int64_t num, const int64_t *idxs, const int64_t *tss,
                            const int64_t *lens, int pad_head, int64_t ofst, int64_t span,
                            int64_t traj_stride, int64_t step_bytes, int64_t col_base,
                            int64_t *src_offsets, int64_t *dst_offsets, int64_t *copy_lens,
                            void *stream) {
  if (num < 0) return GEAR_HIP_EINVAL;
  if (num == 0) return 0;
  if (!idxs || !tss || !lens || !src_offsets || !dst_offsets || !copy_lens) return GEAR_HIP_EINVAL;
  const int64_t blocks = ceil_div64(num, kBlock);
  if (blocks >= 0x7fffffffll) return GEAR_HIP_ERANGE;
  sub_kernel<<<dim3((unsigned)blocks), dim3(kBlock), 0, as_stream(stream)>>>(
      num, idxs, tss, lens, pad_head ? 1 : 0, ofst, span, traj_stride, step_bytes, col_base,
      src_offsets, dst_offsets, copy_lens);
  GEARHIP_RETURN_IF_LAUNCH_FAILED();
  return 0;
}

extern "C" int gear_hip_split_step_index(const int64_t *flat, int64_t num, int64_t trajectory_length,
                                         int64_t modulo, int64_t *idxs, int64_t *tss,
                                         int64_t *lens, void *stream) {
  if (num < 0 || trajectory_length <= 0 || modulo < 0) return GEAR_HIP_EINVAL;
  if (num == 0) return 0;
  if (!flat || !idxs || !tss) return GEAR_HIP_EINVAL;
  const int64_t blocks = ceil_div64(num, kBlock);
  if (blocks >= 0x7fffffffll) return GEAR_HIP_ERANGE;
  split_kernel<<<dim3((unsigned)blocks), dim3(kBlock), 0, as_stream(stream)>>>(
      flat, num, trajectory_length, modulo, idxs, tss, lens);
  GEARHIP_RETURN_IF_LAUNCH_FAILED();
  return 0;
}

extern "C" int gear_hip_take_i64(const int64_t *table, int64_t n, const int64_t *idx, int64_t num,
                                 int64_t add, int64_t *out, void *stream) {
  if (n < 0 || num < 0) return GEAR_HIP_EINVAL;
  if (num == 0) return 0;
  if (!table || !idx || !out) return GEAR_HIP_EINVAL;
  const int64_t blocks = ceil_div64(num, kBlock);
  if (blocks >= 0x7fffffffll) return GEAR_HIP_ERANGE;
  take_kernel<<<dim3((unsigned)blocks), dim3(kBlock), 0, as_stream(stream)>>>(table, n, idx, num,
                                                                             add, out);
  GEARHIP_RETURN_IF_LAUNCH_FAILED();
  return 0;
}
