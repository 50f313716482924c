// fl_device.h -- device-side primitives shared by the scheduler and the copy kernels: wavefront scans built on
// DPP row shifts and row broadcasts (64-wide wavefronts), lane broadcasts and shifts, and the division helpers.
// Everything sits in an unnamed namespace: each translation unit compiles its own copy.
#ifndef FL_DEVICE_H_
#define FL_DEVICE_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "fl_internal.h"

// ------------------------------------------------------------------------------------------------
// wavefront scan primitives (DPP)
// ------------------------------------------------------------------------------------------------
namespace {

constexpr int kWave = 64;
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

// DPP controls of the GFX9 ISA: row_shr:n = 0x110+n, row_bcast:15 = 0x142, row_bcast:31 = 0x143.
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_u32(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xf, 0xf, false);
}
template <int CTRL>
__device__ __forceinline__ uint64_t dpp_u64(uint64_t v) {
  uint32_t lo = dpp_u32<CTRL>((uint32_t)v);
  uint32_t hi = dpp_u32<CTRL>((uint32_t)(v >> 32));
  return ((uint64_t)hi << 32) | lo;
}

// One step of a Hillis-Steele scan: lanes for which `take` holds add the value moved in from below.
#define FL_SCAN_STEP(T, MOVE, CTRL, COND) \
  { T t = MOVE<CTRL>(v); if (COND) v += t; }

// inclusive sum over the 64 lanes of a wavefront
__device__ __forceinline__ uint64_t wave_incl_sum_u64(uint64_t v, int lane) {
  const int r = lane & 15;
  FL_SCAN_STEP(uint64_t, dpp_u64, 0x111, r >= 1)
  FL_SCAN_STEP(uint64_t, dpp_u64, 0x112, r >= 2)
  FL_SCAN_STEP(uint64_t, dpp_u64, 0x114, r >= 4)
  FL_SCAN_STEP(uint64_t, dpp_u64, 0x118, r >= 8)
  FL_SCAN_STEP(uint64_t, dpp_u64, 0x142, (lane & 31) >= 16)
  FL_SCAN_STEP(uint64_t, dpp_u64, 0x143, lane >= 32)
  return v;
}
__device__ __forceinline__ uint32_t wave_incl_sum_u32(uint32_t v, int lane) {
  const int r = lane & 15;
  FL_SCAN_STEP(uint32_t, dpp_u32, 0x111, r >= 1)
  FL_SCAN_STEP(uint32_t, dpp_u32, 0x112, r >= 2)
  FL_SCAN_STEP(uint32_t, dpp_u32, 0x114, r >= 4)
  FL_SCAN_STEP(uint32_t, dpp_u32, 0x118, r >= 8)
  FL_SCAN_STEP(uint32_t, dpp_u32, 0x142, (lane & 31) >= 16)
  FL_SCAN_STEP(uint32_t, dpp_u32, 0x143, lane >= 32)
  return v;
}
#undef FL_SCAN_STEP

// Segmented inclusive sum: f marks "a segment starts at or before me inside my own span"; the
// combine is (f1,v1)+(f2,v2) = (f1|f2, f2 ? v2 : v1+v2) with operand 1 the lower lanes.
#define FL_SEG_STEP(CTRL, COND)                                   \
  {                                                               \
    uint64_t tv = dpp_u64<CTRL>(v);                               \
    uint32_t tf = dpp_u32<CTRL>(f);                               \
    if (COND) { if (!f) v += tv; f |= tf; }                       \
  }
__device__ __forceinline__ void wave_incl_segsum_u64(uint64_t& v, uint32_t& f, int lane) {
  const int r = lane & 15;
  FL_SEG_STEP(0x111, r >= 1)
  FL_SEG_STEP(0x112, r >= 2)
  FL_SEG_STEP(0x114, r >= 4)
  FL_SEG_STEP(0x118, r >= 8)
  FL_SEG_STEP(0x142, (lane & 31) >= 16)
  FL_SEG_STEP(0x143, lane >= 32)
}
#undef FL_SEG_STEP

__device__ __forceinline__ uint64_t bcast_lane_u64(uint64_t v, int src_lane) {
  uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)v, src_lane);
  uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(v >> 32), src_lane);
  return ((uint64_t)hi << 32) | lo;
}
__device__ __forceinline__ uint32_t bcast_lane_u32(uint32_t v, int src_lane) {
  return (uint32_t)__builtin_amdgcn_readlane((int)v, src_lane);
}

// value of the lane below (lane 0 gets 0): turns an inclusive scan into an exclusive one
__device__ __forceinline__ uint64_t wave_shift_up_u64(uint64_t v, int lane) {
  // wave_shr:1 does not exist on every GFX9 part for 64 lanes; go through a bpermute
  int src = (lane - 1) << 2;
  uint32_t lo = (uint32_t)__builtin_amdgcn_ds_bpermute(src, (int)(uint32_t)v);
  uint32_t hi = (uint32_t)__builtin_amdgcn_ds_bpermute(src, (int)(uint32_t)(v >> 32));
  uint64_t r = ((uint64_t)hi << 32) | lo;
  return lane == 0 ? 0 : r;
}
__device__ __forceinline__ uint32_t wave_shift_up_u32(uint32_t v, int lane) {
  uint32_t r = (uint32_t)__builtin_amdgcn_ds_bpermute((lane - 1) << 2, (int)v);
  return lane == 0 ? 0 : r;
}

// 64-bit division is a long software routine on this ISA and almost every operand here fits 32
// bits; the wide case is kept out of line so that the kernel stays small enough for the
// instruction cache (a lone wavefront cannot hide instruction fetch).
__device__ __attribute__((noinline)) uint64_t div_u64_wide(uint64_t a, uint64_t b) { return a / b; }
__device__ __forceinline__ uint64_t div_u64(uint64_t a, uint64_t b) {
  return ((a | b) >> 32) == 0 ? (uint64_t)((uint32_t)a / (uint32_t)b) : div_u64_wide(a, b);
}
__device__ __forceinline__ uint64_t mod_u64(uint64_t a, uint64_t b) {
  return ((a | b) >> 32) == 0 ? (uint64_t)((uint32_t)a % (uint32_t)b) : a - div_u64_wide(a, b) * b;
}

// A kernel's argument block is read with scalar loads, and the compiler places each load next to its first use:
// behind every branch waits another round trip to memory that the host wrote a moment ago and no cache holds
// yet.  Reading one word of every 64-byte line of the block first, all in flight together, turns that chain
// of misses into one miss plus scalar-cache hits.
// Workgroups of a launch are handed to the eight XCDs in turn: workgroup b runs on XCD b mod 8, so with tile = b every
// XCD touches every eighth tile of the stream.  xcd_tile() gives each XCD runs of 32 consecutive tiles instead (1 MiB
// at 32 KiB tiles): workgroups 256 k .. 256 k + 255 still cover tiles 256 k .. 256 k + 255, but XCD x takes
// 256 k + 32 x .. 256 k + 32 x + 31.  On plain copies this takes 3-5 % less time, inside the Infinity Cache and
// beyond it (64 MiB: 20.1 -> 19.2 us, 1 GiB: 386 -> 360 us; runs of 4 or 256 tiles gain half as much or nothing).
// `full` is the workgroup count rounded down to a multiple of 256 (0 switches the mapping off); workgroups from
// there on keep tile = b, so the map is a permutation of the grid (on a partition of the GPU that hands workgroups out
// differently it stays one, and only the gain is lost).
// Bit 5 of `full` (free: full is a multiple of 256) asks for the other extreme instead, for experiments: XCD x takes the
// x-th eighth of the tiles front to back, so that the eight XCDs work in eight places of the stream that lie far apart.
constexpr uint32_t kXcdEighths = 32u;
__device__ __forceinline__ uint32_t xcd_tile(uint32_t b, uint32_t full) {
  const uint32_t n = full & ~(kXcdBlock - 1);
  if (full & kXcdEighths) return b < n ? (b & 7u) * (n >> 3) + (b >> 3) : b;
  return b < n ? (b & ~(kXcdBlock - 1)) + ((b & 7u) << kXcdRunShift) + ((b >> 3) & ((1u << kXcdRunShift) - 1)) : b;
}
// The same for a grid (tiles of a chunk, chunks) whose width is a power of two: xcd_map = full | log2(width).
// Takes the workgroup's place in the grid, returns the tile of the chunk (x) and the chunk (y) it works on.
__device__ __forceinline__ void xcd_tile_2d(uint32_t xcd_map, uint32_t& x, uint32_t& y) {
  if (xcd_map == 0) return;
  const uint32_t sh = xcd_map & 31u;
  const uint32_t t = xcd_tile((y << sh) + x, xcd_map & ~31u);
  x = t & ((1u << sh) - 1);
  y = t >> sh;
}

template <class Args>
__device__ __forceinline__ void warm_kernel_args(const Args& a) {
  const uint32_t* p = reinterpret_cast<const uint32_t*>(&a);
  constexpr int kDwords = (int)(sizeof(Args) / 4);
  uint32_t z = p[kDwords - 1];
#pragma unroll
  for (int i = 0; i < kDwords; i += 16) z |= p[i];
  asm volatile("" ::"s"(z));
}

}  // namespace

#endif  // FL_DEVICE_H_
