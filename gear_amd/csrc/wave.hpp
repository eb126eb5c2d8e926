// Wave64 primitives for gfx950 built on DPP row shifts / broadcasts and ballots.
#pragma once
#include "common.hpp"

namespace gearhip {

// DPP controls (GFX9 encoding)
constexpr int kDppRowShr1 = 0x111;
constexpr int kDppRowShr2 = 0x112;
constexpr int kDppRowShr4 = 0x114;
constexpr int kDppRowShr8 = 0x118;
constexpr int kDppRowBcast15 = 0x142;  // lane 15 of each row -> every lane of the next row
constexpr int kDppRowBcast31 = 0x143;  // lane 31 -> every lane of rows 2 and 3
constexpr int kDppWaveShr1 = 0x138;     // lane i-1 -> lane i across the whole wave

// Value of lane (i - shift) moved into lane i; lanes without a source (or whose row is disabled
// by ROW_MASK) receive 0.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ int dpp_i32(int x) {
  return __builtin_amdgcn_update_dpp(0, x, CTRL, ROW_MASK, 0xf, false);
}

template <int CTRL, int ROW_MASK>
__device__ __forceinline__ double dpp_f64(double x) {
  int lo = __double2loint(x), hi = __double2hiint(x);
  lo = dpp_i32<CTRL, ROW_MASK>(lo);
  hi = dpp_i32<CTRL, ROW_MASK>(hi);
  return __hiloint2double(hi, lo);
}

template <int CTRL, int ROW_MASK>
__device__ __forceinline__ int64_t dpp_i64(int64_t x) {
  int lo = (int)(uint32_t)x, hi = (int)(uint32_t)((uint64_t)x >> 32);
  lo = dpp_i32<CTRL, ROW_MASK>(lo);
  hi = dpp_i32<CTRL, ROW_MASK>(hi);
  return (int64_t)(((uint64_t)(uint32_t)hi << 32) | (uint32_t)lo);
}

// Inclusive scan (sum) over the 64 lanes of a wave.  All 64 lanes must be active.
__device__ __forceinline__ double wave_inclusive_sum(double x) {
  x += dpp_f64<kDppRowShr1, 0xf>(x);
  x += dpp_f64<kDppRowShr2, 0xf>(x);
  x += dpp_f64<kDppRowShr4, 0xf>(x);
  x += dpp_f64<kDppRowShr8, 0xf>(x);
  x += dpp_f64<kDppRowBcast15, 0xa>(x);
  x += dpp_f64<kDppRowBcast31, 0xc>(x);
  return x;
}

__device__ __forceinline__ int64_t wave_inclusive_sum(int64_t x) {
  x += dpp_i64<kDppRowShr1, 0xf>(x);
  x += dpp_i64<kDppRowShr2, 0xf>(x);
  x += dpp_i64<kDppRowShr4, 0xf>(x);
  x += dpp_i64<kDppRowShr8, 0xf>(x);
  x += dpp_i64<kDppRowBcast15, 0xa>(x);
  x += dpp_i64<kDppRowBcast31, 0xc>(x);
  return x;
}

__device__ __forceinline__ int wave_inclusive_sum(int x) {
  x += dpp_i32<kDppRowShr1, 0xf>(x);
  x += dpp_i32<kDppRowShr2, 0xf>(x);
  x += dpp_i32<kDppRowShr4, 0xf>(x);
  x += dpp_i32<kDppRowShr8, 0xf>(x);
  x += dpp_i32<kDppRowBcast15, 0xa>(x);
  x += dpp_i32<kDppRowBcast31, 0xc>(x);
  return x;
}

// Exclusive scan from an inclusive one: the value of the previous lane, 0 in lane 0.
__device__ __forceinline__ double wave_shift_up1(double x) { return dpp_f64<kDppWaveShr1, 0xf>(x); }
__device__ __forceinline__ int64_t wave_shift_up1(int64_t x) { return dpp_i64<kDppWaveShr1, 0xf>(x); }
__device__ __forceinline__ int wave_shift_up1(int x) { return dpp_i32<kDppWaveShr1, 0xf>(x); }

__device__ __forceinline__ int lane_id() { return (int)__lane_id(); }

// Value held by lane `src` (uniform) of the calling wave.
__device__ __forceinline__ double wave_read_lane(double x, int src) {
  int lo = __builtin_amdgcn_readlane(__double2loint(x), src);
  int hi = __builtin_amdgcn_readlane(__double2hiint(x), src);
  return __hiloint2double(hi, lo);
}
__device__ __forceinline__ int64_t wave_read_lane(int64_t x, int src) {
  uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)x, src);
  uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)((uint64_t)x >> 32), src);
  return (int64_t)(((uint64_t)hi << 32) | lo);
}
__device__ __forceinline__ int wave_read_lane(int x, int src) {
  return __builtin_amdgcn_readlane(x, src);
}

// Sum over the wave, returned in every lane.
template <typename T>
__device__ __forceinline__ T wave_sum(T x) {
  return wave_read_lane(wave_inclusive_sum(x), kWave - 1);
}

__device__ __forceinline__ uint64_t wave_ballot(bool p) { return __ballot(p); }

// Agent-scope relaxed 64-bit accesses: they reach the device-coherent level, so a word written
// by a workgroup on one XCD is seen by workgroups on the others without further fences.
__device__ __forceinline__ uint64_t load_agent(const uint64_t *p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void store_agent(uint64_t *p, uint64_t v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

}  // namespace gearhip
