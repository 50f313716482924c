// fl_copy.hip -- the byte movers and their entry points:
//   * fl_copy_uniform_fused : scheduling and copy in one launch (uniform split, one credit row), also for a batch of requests
//   * fl_copy_uniform       : table-driven stripe / reassemble for a uniform split (2-D grid)
//   * fl_copy_tiles         : the same for any table (tile -> row by a wavefront search)
//   * fl_page_tiles         : paged gather / scatter (non-contiguous pages <-> lane windows)
//   * fl_plain_copy         : calibration copy with the same inner loop
// The path is an HBM-bound byte mover; nothing here contracts, so no MFMA.
#include <cstring>
#include <new>
#include <type_traits>
#include <vector>

#include "fl_closed_form.h"
#include "fl_device.h"
#include "fl_launch.h"

namespace {

// ------------------------------------------------------------------------------------------------
// copy kernels
// ------------------------------------------------------------------------------------------------

constexpr int kCopyBlock = 256;
constexpr int kCopyUnroll = 8;

// Streaming mode of a copy.  Bits 0 and 1: nontemporal loads, nontemporal stores.  Bits 2 and 3 (the lane engine's
// workers, which never leave the GPU and so have no kernel boundary to make their accesses coherent): stores, loads at
// system scope.  Such a load is served from memory rather than from a line that an L1 or this XCD's L2 has kept, and
// such a store is written through to memory and is there once the wave's memory counter has run down, so a workgroup
// that touches memory in no other way needs neither a cache invalidate before its loads nor an L2 write-back behind
// its stores.  Sixteen-byte accesses take a cache policy only as buffer accesses (the compiler makes atomics of eight
// bytes at most, and eight-byte stores cost a quarter of the engine's rate), so in these modes a copy addresses its
// operands through buffer resources.
template <int NT>
__device__ __forceinline__ u32x4 ld16(const u32x4* p) {
  return (NT & 1) ? __builtin_nontemporal_load(p) : *p;
}
template <int NT>
__device__ __forceinline__ void st16(u32x4* p, u32x4 v) {
  if (NT & 2) __builtin_nontemporal_store(v, p); else *p = v;
}
constexpr int kAuxSystemScope = 1 | 16;   // cache policy of a buffer access: sc0 | sc1
struct NoBuffer {};
// A raw buffer over [base, base + bytes): byte offsets, accesses past the end dropped by the hardware.  The base is the
// same in every lane (a copy's operands are the workgroup's); reading it from the first lane tells the compiler so.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t system_buffer(const void* base, uint32_t bytes) {
  const uint64_t a = (uint64_t)base;
  // (the builtin returns a signed int: through uint32_t, or a low half with its top bit set would smear over the high half)
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)a), hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)(a >> 32));
  const uint64_t u = (uint64_t)lo | ((uint64_t)hi << 32);
  return __builtin_amdgcn_make_buffer_rsrc((void*)u, 0, (int)bytes, 0x00020000);
}
// the sixteen-byte vectors of a copy's source and destination
template <int NT>
struct VecIn {
  const u32x4* s;
  [[no_unique_address]] std::conditional_t<(NT & 8) != 0, __amdgpu_buffer_rsrc_t, NoBuffer> r;
  __device__ __forceinline__ VecIn(const u32x4* s_, uint32_t vectors) : s(s_) {
    if constexpr (NT & 8) r = system_buffer(s_, vectors * 16);
  }
  __device__ __forceinline__ u32x4 operator()(uint32_t idx) const {
    if constexpr (NT & 8) return __builtin_amdgcn_raw_buffer_load_b128(r, (int)(idx * 16), 0, kAuxSystemScope);
    else return ld16<NT>(s + idx);
  }
};
template <int NT>
struct VecOut {
  u32x4* d;
  [[no_unique_address]] std::conditional_t<(NT & 4) != 0, __amdgpu_buffer_rsrc_t, NoBuffer> r;
  __device__ __forceinline__ VecOut(u32x4* d_, uint32_t vectors) : d(d_) {
    if constexpr (NT & 4) r = system_buffer(d_, vectors * 16);
  }
  __device__ __forceinline__ void operator()(uint32_t idx, u32x4 v) const {
    if constexpr (NT & 4) __builtin_amdgcn_raw_buffer_store_b128(v, r, (int)(idx * 16), 0, kAuxSystemScope);
    else st16<NT>(d + idx, v);
  }
};
template <int NT>
__device__ __forceinline__ void copy1(uint8_t* d, const uint8_t* s) {
  uint8_t v;
  if constexpr (NT & 8) v = __hip_atomic_load(s, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM); else v = *s;
  if constexpr (NT & 4) __hip_atomic_store(d, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM); else *d = v;
}
// a small object (table row, header field, status word) stored whole, or in mode 4 as 4- or 8-byte system-scope pieces
template <int NT, class T>
__device__ __forceinline__ void st_obj(T* p, const T& v) {
  if constexpr (NT & 4) {
    if constexpr (sizeof(T) % 8 == 0 && alignof(T) >= 8) {
      uint64_t w[sizeof(T) / 8];
      __builtin_memcpy(w, &v, sizeof(T));
#pragma unroll
      for (uint32_t i = 0; i < sizeof(T) / 8; ++i) __hip_atomic_store((uint64_t*)p + i, w[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    } else {
      static_assert(sizeof(T) % 4 == 0 && alignof(T) >= 4, "whole words");
      uint32_t w[sizeof(T) / 4];
      __builtin_memcpy(w, &v, sizeof(T));
#pragma unroll
      for (uint32_t i = 0; i < sizeof(T) / 4; ++i) __hip_atomic_store((uint32_t*)p + i, w[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    }
  } else {
    *p = v;
  }
}

template <int NT, int U>
__device__ __forceinline__ void copy_exact(u32x4* __restrict__ d, const u32x4* __restrict__ s, uint32_t tid) {
  u32x4 r[U];
#pragma unroll
  for (int j = 0; j < U; ++j) r[j] = ld16<NT>(s + j * kCopyBlock + tid);
#pragma unroll
  for (int j = 0; j < U; ++j) st16<NT>(d + j * kCopyBlock + tid, r[j]);
}

// Source and destination misaligned differently (exactly packed windows make that the ordinary case for chunk sizes
// that are no multiple of 16): the destination is written in aligned 16-byte vectors, each put together from the two
// aligned source vectors it straddles.  A thread loads only the first of the two; the second is the first of the thread
// one lane up (consecutive threads copy consecutive vectors) and comes over with a wavefront shift (DPP wave_shl:1),
// except in the wavefront's last lane, which loads it.  Both source vectors hold bytes of the copy, so no load leaves the
// pages the source occupies.  The byte shift is a dword select (shift / 4, the same for the whole workgroup) and a
// v_alignbyte_b32 per dword.  Measured against the alternatives on 850 MiB of odd-sized blocks: two aligned loads per
// thread 467 + 463 us, unaligned 16-byte loads (the memory pipeline takes them) 346 + 411 us, aligned copies 287 + 285 us.
__device__ __forceinline__ uint32_t lane_above(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x130 /* wave_shl:1 */, 0xf, 0xf, false);
}
__device__ __forceinline__ u32x4 funnel16(u32x4 a, u32x4 b, uint32_t q, uint32_t r) {
  uint32_t w0, w1, w2, w3, w4;
  switch (q) {
    case 0: w0 = a.x; w1 = a.y; w2 = a.z; w3 = a.w; w4 = b.x; break;
    case 1: w0 = a.y; w1 = a.z; w2 = a.w; w3 = b.x; w4 = b.y; break;
    case 2: w0 = a.z; w1 = a.w; w2 = b.x; w3 = b.y; w4 = b.z; break;
    default: w0 = a.w; w1 = b.x; w2 = b.y; w3 = b.z; w4 = b.w; break;
  }
  u32x4 o;
  o.x = __builtin_amdgcn_alignbyte(w1, w0, r);
  o.y = __builtin_amdgcn_alignbyte(w2, w1, r);
  o.z = __builtin_amdgcn_alignbyte(w3, w2, r);
  o.w = __builtin_amdgcn_alignbyte(w4, w3, r);
  return o;
}
template <int NT>
__device__ __forceinline__ void block_copy_shifted(uint8_t* __restrict__ dst, const uint8_t* __restrict__ src, uint32_t bytes, uint32_t tid) {
  uint32_t head = (uint32_t)((16 - ((uintptr_t)dst & 15)) & 15);
  if (head > bytes) head = bytes;
  if (tid < head) dst[tid] = src[tid];
  const uint32_t nvec = (bytes - head) >> 4;
  const uintptr_t s0 = (uintptr_t)(src + head);
  const uint32_t shift = (uint32_t)(s0 & 15);          // 1..15: the two sides differ in their alignment
  const uint32_t q = shift >> 2, r = shift & 3;
  const u32x4* s = (const u32x4*)(s0 - shift);         // aligned vector i holds the first bytes of destination vector i
  u32x4* d = (u32x4*)(dst + head);
  const bool top = (tid & (kWave - 1)) == kWave - 1;
  for (uint32_t b = 0; b < nvec; b += kCopyBlock * kCopyUnroll) {
    u32x4 lo[kCopyUnroll], hi[kCopyUnroll];
#pragma unroll
    for (int j = 0; j < kCopyUnroll; ++j) {
      const uint32_t idx = b + j * kCopyBlock + tid;
      if (idx <= nvec) lo[j] = ld16<NT>(s + idx);      // vector nvec is the second half of the last destination vector
      if (top && idx < nvec) hi[j] = ld16<NT>(s + idx + 1);
    }
#pragma unroll
    for (int j = 0; j < kCopyUnroll; ++j) {
      const uint32_t idx = b + j * kCopyBlock + tid;
      u32x4 up;
      up.x = lane_above(lo[j].x);
      up.y = lane_above(lo[j].y);
      up.z = lane_above(lo[j].z);
      up.w = lane_above(lo[j].w);
      if (top) up = hi[j];
      if (idx < nvec) st16<NT>(d + idx, funnel16(lo[j], up, q, r));
    }
  }
  const uint32_t tail0 = head + (nvec << 4);
  const uint32_t tail = bytes - tail0;
  if (tid < tail) dst[tail0 + tid] = src[tail0 + tid];
}

// ---- the same copies in the system-scope modes (bits 2 and 3): vectors through buffer resources, bytes as atomics ----
// (A second set of routines rather than the first one over accessors: addressing by index off a base instead of by
// pointer changes the launched kernels' address arithmetic and instruction order, and their code is left as tuned.)
template <int NT, int U>
__device__ __forceinline__ void copy_exact_system(const VecOut<NT>& out, const VecIn<NT>& in, uint32_t tid) {
  u32x4 r[U];
#pragma unroll
  for (int j = 0; j < U; ++j) r[j] = in(j * kCopyBlock + tid);
#pragma unroll
  for (int j = 0; j < U; ++j) out(j * kCopyBlock + tid, r[j]);
}

template <int NT>
__device__ __forceinline__ void block_copy_shifted_system(uint8_t* __restrict__ dst, const uint8_t* __restrict__ src, uint32_t bytes, uint32_t tid) {
  uint32_t head = (uint32_t)((16 - ((uintptr_t)dst & 15)) & 15);
  if (head > bytes) head = bytes;
  if (tid < head) copy1<NT>(dst + tid, src + tid);
  const uint32_t nvec = (bytes - head) >> 4;
  const uintptr_t s0 = (uintptr_t)(src + head);
  const uint32_t shift = (uint32_t)(s0 & 15);          // 1..15: the two sides differ in their alignment
  const uint32_t q = shift >> 2, r = shift & 3;
  const VecIn<NT> in((const u32x4*)(s0 - shift), nvec + 1);   // aligned vector i holds the first bytes of destination vector i
  const VecOut<NT> out((u32x4*)(dst + head), nvec);
  const bool top = (tid & (kWave - 1)) == kWave - 1;
  for (uint32_t b = 0; b < nvec; b += kCopyBlock * kCopyUnroll) {
    u32x4 lo[kCopyUnroll], hi[kCopyUnroll];
#pragma unroll
    for (int j = 0; j < kCopyUnroll; ++j) {
      const uint32_t idx = b + j * kCopyBlock + tid;
      if (idx <= nvec) lo[j] = in(idx);                // vector nvec is the second half of the last destination vector
      if (top && idx < nvec) hi[j] = in(idx + 1);
    }
#pragma unroll
    for (int j = 0; j < kCopyUnroll; ++j) {
      const uint32_t idx = b + j * kCopyBlock + tid;
      u32x4 up;
      up.x = lane_above(lo[j].x);
      up.y = lane_above(lo[j].y);
      up.z = lane_above(lo[j].z);
      up.w = lane_above(lo[j].w);
      if (top) up = hi[j];
      if (idx < nvec) out(idx, funnel16(lo[j], up, q, r));
    }
  }
  const uint32_t tail0 = head + (nvec << 4);
  const uint32_t tail = bytes - tail0;
  if (tid < tail) copy1<NT>(dst + tail0 + tid, src + tail0 + tid);
}

template <int NT>
__device__ __forceinline__ void block_copy_system(uint8_t* __restrict__ dst, const uint8_t* __restrict__ src,
                                           uint32_t bytes) {
  const uint32_t tid = threadIdx.x;
  const uintptr_t sa = (uintptr_t)src, da = (uintptr_t)dst;
  if (((sa ^ da) & 15) != 0) {
    block_copy_shifted_system<NT>(dst, src, bytes, tid);
    return;
  }
  uint32_t head = (uint32_t)((16 - (sa & 15)) & 15);
  if (head > bytes) head = bytes;
  if (tid < head) copy1<NT>(dst + tid, src + tid);
  const uint32_t body = bytes - head;
  const uint32_t nvec = body >> 4;
  const VecIn<NT> in((const u32x4*)(src + head), nvec);
  const VecOut<NT> out((u32x4*)(dst + head), nvec);
  // whole tiles of the usual sizes: every load of the tile is issued before the first store, unpredicated
  if (nvec == kCopyBlock * 16) { copy_exact_system<NT, 16>(out, in, tid); }
  else if (nvec == kCopyBlock * 8) { copy_exact_system<NT, 8>(out, in, tid); }
  else if (nvec == kCopyBlock * 4) { copy_exact_system<NT, 4>(out, in, tid); }
  else {
    for (uint32_t b = 0; b < nvec; b += kCopyBlock * kCopyUnroll) {
      u32x4 r[kCopyUnroll];
#pragma unroll
      for (int j = 0; j < kCopyUnroll; ++j) {
        const uint32_t idx = b + j * kCopyBlock + tid;
        if (idx < nvec) r[j] = in(idx);
      }
#pragma unroll
      for (int j = 0; j < kCopyUnroll; ++j) {
        const uint32_t idx = b + j * kCopyBlock + tid;
        if (idx < nvec) out(idx, r[j]);
      }
    }
  }
  const uint32_t tail0 = head + (nvec << 4);
  const uint32_t tail = bytes - tail0;
  if (tid < tail) copy1<NT>(dst + tail0 + tid, src + tail0 + tid);
}

// Copies `bytes` from src to dst with the whole workgroup.  Fast path: both 16-byte aligned ->
// dwordx4 loads batched kCopyUnroll deep before the stores.  Equal misalignment: byte head up to
// the boundary, vectors, byte tail.  Different misalignment: aligned vector stores, each merged from two aligned source vectors.
template <int NT>
__device__ __forceinline__ void block_copy(uint8_t* __restrict__ dst, const uint8_t* __restrict__ src,
                                           uint32_t bytes) {
  if constexpr ((NT & 12) != 0) {
    block_copy_system<NT>(dst, src, bytes);
    return;
  }
  const uint32_t tid = threadIdx.x;
  const uintptr_t sa = (uintptr_t)src, da = (uintptr_t)dst;
  if (((sa ^ da) & 15) != 0) {
    block_copy_shifted<NT>(dst, src, bytes, tid);
    return;
  }
  uint32_t head = (uint32_t)((16 - (sa & 15)) & 15);
  if (head > bytes) head = bytes;
  if (tid < head) dst[tid] = src[tid];
  const uint32_t body = bytes - head;
  const uint32_t nvec = body >> 4;
  const u32x4* s = (const u32x4*)(src + head);
  u32x4* d = (u32x4*)(dst + head);
  // whole tiles of the usual sizes: every load of the tile is issued before the first store, unpredicated
  if (nvec == kCopyBlock * 16) { copy_exact<NT, 16>(d, s, tid); }
  else if (nvec == kCopyBlock * 8) { copy_exact<NT, 8>(d, s, tid); }
  else if (nvec == kCopyBlock * 4) { copy_exact<NT, 4>(d, s, tid); }
  else {
    for (uint32_t b = 0; b < nvec; b += kCopyBlock * kCopyUnroll) {
      u32x4 r[kCopyUnroll];
#pragma unroll
      for (int j = 0; j < kCopyUnroll; ++j) {
        const uint32_t idx = b + j * kCopyBlock + tid;
        if (idx < nvec) r[j] = ld16<NT>(s + idx);
      }
#pragma unroll
      for (int j = 0; j < kCopyUnroll; ++j) {
        const uint32_t idx = b + j * kCopyBlock + tid;
        if (idx < nvec) st16<NT>(d + idx, r[j]);
      }
    }
  }
  const uint32_t tail0 = head + (nvec << 4);
  const uint32_t tail = bytes - tail0;
  if (tid < tail) dst[tail0 + tid] = src[tail0 + tid];
}

// One source, two destinations: every vector is loaded once and stored twice (staging window and the wire's far end,
// or staging window and receive buffer), so the second copy costs no second read and no barrier between a workgroup's
// store and its re-load.  When the three addresses are not equally aligned the bytes are copied twice from the source.
// NT is the streaming mode of the loads and of the stores to d1, NT2's store bits that of the stores to d2.
template <int NT, int NT2, int U>
__device__ __forceinline__ void copy2_exact(const VecOut<NT>& out1, const VecOut<NT2>& out2, const VecIn<NT>& in, uint32_t tid) {
  u32x4 r[U];
#pragma unroll
  for (int j = 0; j < U; ++j) r[j] = in(j * kCopyBlock + tid);
#pragma unroll
  for (int j = 0; j < U; ++j) out1(j * kCopyBlock + tid, r[j]);
#pragma unroll
  for (int j = 0; j < U; ++j) out2(j * kCopyBlock + tid, r[j]);
  // The stores above must stay in this block.  Left to itself the optimizer sinks the trailing stores of this path and
  // of the predicated loop beside it into one shared block with the vector index as a phi, and the backend then left
  // the index of the first store undefined on this path (seen in the generated code, and on the GPU as a lost or a wild
  // store).  A marker that differs from path to path keeps the paths' tails apart.
  asm volatile("; two-destination copy, %0 vectors per thread" ::"n"(U) : "memory");
}
template <int NT, int NT2>
__device__ __forceinline__ void block_copy2(uint8_t* d1, uint8_t* d2, const uint8_t* src, uint32_t bytes) {
  const uintptr_t sa = (uintptr_t)src;
  if ((((sa ^ (uintptr_t)d1) | (sa ^ (uintptr_t)d2)) & 15) != 0) {
    block_copy<NT>(d1, src, bytes);
    block_copy<NT2>(d2, src, bytes);
    return;
  }
  const uint32_t tid = threadIdx.x;
  uint32_t head = (uint32_t)((16 - (sa & 15)) & 15);
  if (head > bytes) head = bytes;
  if (tid < head) { copy1<NT>(d1 + tid, src + tid); copy1<NT2>(d2 + tid, src + tid); }
  const uint32_t nvec = (bytes - head) >> 4;
  const VecIn<NT> in((const u32x4*)(src + head), nvec);
  const VecOut<NT> out1((u32x4*)(d1 + head), nvec);
  const VecOut<NT2> out2((u32x4*)(d2 + head), nvec);
  // whole tiles of the usual sizes (one tile, a share of two): every load is issued before the first store, unpredicated
  if (nvec == kCopyBlock * 16) { copy2_exact<NT, NT2, 16>(out1, out2, in, tid); }
  else if (nvec == kCopyBlock * 8) { copy2_exact<NT, NT2, 8>(out1, out2, in, tid); }
  else {
    for (uint32_t b = 0; b < nvec; b += kCopyBlock * kCopyUnroll) {
      u32x4 r[kCopyUnroll];
#pragma unroll
      for (int j = 0; j < kCopyUnroll; ++j) {
        const uint32_t idx = b + j * kCopyBlock + tid;
        r[j] = idx < nvec ? in(idx) : u32x4{0, 0, 0, 0};
      }
#pragma unroll
      for (int j = 0; j < kCopyUnroll; ++j) {
        const uint32_t idx = b + j * kCopyBlock + tid;
        if (idx < nvec) out1(idx, r[j]);
      }
#pragma unroll
      for (int j = 0; j < kCopyUnroll; ++j) {
        const uint32_t idx = b + j * kCopyBlock + tid;
        if (idx < nvec) out2(idx, r[j]);
      }
      asm volatile("; two-destination copy, predicated" ::: "memory");   // (see copy2_exact)
    }
  }
  const uint32_t tail0 = head + (nvec << 4);
  const uint32_t tail = bytes - tail0;
  if (tid < tail) { copy1<NT>(d1 + tail0 + tid, src + tail0 + tid); copy1<NT2>(d2 + tail0 + tid, src + tail0 + tid); }
}

struct CopyArgs {
  uint8_t* user;
  uint64_t user_bytes;
  flh_windows win;
  const flh_chunk_desc* table;
  const flh_sched_hdr* hdr;
  int32_t* status;
  uint32_t n_chunks_max;
  uint32_t tile_bytes;
  // header fields the host already knows (has_hint != 0): saves one dependent memory round trip
  uint32_t has_hint, hint_total_tiles, hint_n_chunks, hint_uniform_tiles;
  uint32_t xcd;   // xcd_tile()'s `full` (fl_copy_tiles, one workgroup per tile) or xcd_tile_2d()'s map (fl_copy_uniform); 0 = off
};

// Row of the table that owns copy tile t: the last row with tile_base <= t (rows of empty chunks own
// no tile and are stepped over).  A uniform split is answered by one division and one row load; any
// other table by a 64-ary search in which every lane of the wavefront probes one row per round
// (three rounds cover 262144 chunks).  The result is wavefront-uniform.
__device__ __forceinline__ uint32_t find_row(const flh_chunk_desc* __restrict__ table, uint32_t n, uint32_t t,
                                             uint32_t uniform_tiles, uint32_t tile_bytes) {
  if (uniform_tiles) {
    const uint32_t c = t / uniform_tiles;
    if (c < n) {
      const uint32_t tb = table[c].tile_base;
      const uint32_t len = table[c].len;
      if (t >= tb && (uint64_t)(t - tb) * tile_bytes < len) return c;
    }
  }
  const uint32_t lane = threadIdx.x & (kWave - 1);
  uint32_t lo = 0, cnt = n;  // the answer lies in [lo, lo + cnt); table[lo].tile_base <= t
  while (cnt > 1) {
    const uint32_t step = (cnt + kWave - 1) / kWave;
    const uint32_t idx = lo + lane * step;
    const bool le = idx < lo + cnt && table[idx].tile_base <= t;
    const uint32_t k = (uint32_t)__builtin_popcountll(__builtin_amdgcn_ballot_w64(le));
    const uint32_t adv = (k ? k - 1 : 0) * step;
    const uint32_t end = lo + cnt;
    lo += adv;
    cnt = end - lo < step ? end - lo : step;
  }
  return lo;
}

// DIR 0: user -> windows (stripe).  DIR 1: windows -> user (reassemble).
template <int DIR, int NT>
__global__ __launch_bounds__(kCopyBlock) void fl_copy_tiles(CopyArgs a) {
  warm_kernel_args(a);
  const uint32_t total = a.has_hint ? a.hint_total_tiles : a.hdr->total_tiles;
  const uint32_t uniform_tiles = a.has_hint ? a.hint_uniform_tiles : a.hdr->uniform_tiles;
  uint32_t n = a.has_hint ? a.hint_n_chunks : a.hdr->n_chunks;
  if (n > a.n_chunks_max) n = a.n_chunks_max;
  if (n == 0) return;
  for (uint32_t t = xcd_tile(blockIdx.x, a.xcd); t < total; t += gridDim.x) {
    const uint32_t c = find_row(a.table, n, t, uniform_tiles, a.tile_bytes);
    const flh_chunk_desc d = a.table[c];
    const uint64_t off = (uint64_t)(t - d.tile_base) * a.tile_bytes;
    if (t < d.tile_base || off >= d.len) continue;
    const uint32_t bytes = (uint32_t)((d.len - off) < a.tile_bytes ? (d.len - off) : a.tile_bytes);
    // refuse anything that would leave the user buffer or the mapped part of the window
    bool ok = d.lane < a.win.n_lanes;
    if (ok) ok = d.win_off + d.len <= a.win.cap[d.lane] && d.src_off + d.len <= a.user_bytes;
    if (!ok) {
      if (threadIdx.x == 0) *a.status = FLH_E_RANGE;
      continue;
    }
    uint8_t* u = a.user + d.src_off + off;
    uint8_t* w = (uint8_t*)a.win.base[d.lane] + d.win_off + off;
    if (DIR == 0) block_copy<NT>(w, u, bytes); else block_copy<NT>(u, w, bytes);
  }
}

// Any table, expanded beforehand to one descriptor per tile: the workgroup's descriptor is the only thing it waits
// for before its data (the header, where the host has no copy of it, is read alongside, not before).
struct DescArgs {
  uint8_t* user;
  uint64_t user_bytes;
  flh_windows win;
  const flh_tile_desc* tiles;
  const flh_sched_hdr* hdr;
  int32_t* status;
  uint32_t tiles_cap;
  uint32_t has_hint, hint_total_tiles;
  uint32_t xcd;   // xcd_tile()'s `full`; 0 = off
};

template <int DIR, int NT>
__global__ __launch_bounds__(kCopyBlock) void fl_copy_desc(DescArgs a) {
  warm_kernel_args(a);
  const uint32_t t = xcd_tile(blockIdx.x, a.xcd);
  const flh_tile_desc d = a.tiles[t];
  const uint32_t total = a.has_hint ? a.hint_total_tiles : a.hdr->total_tiles;
  if (total > a.tiles_cap) {   // the table did not fit the descriptor array: nothing of it can be trusted
    if (t == 0 && threadIdx.x == 0) *a.status = FLH_E_RANGE;
    return;
  }
  if (t >= total || d.len == 0) return;
  bool ok = d.lane < a.win.n_lanes;
  if (ok) ok = d.win_off + d.len <= a.win.cap[d.lane] && d.src_off + d.len <= a.user_bytes;
  if (!ok) {
    if (threadIdx.x == 0) *a.status = FLH_E_RANGE;
    return;
  }
  uint8_t* u = a.user + d.src_off;
  uint8_t* w = (uint8_t*)a.win.base[d.lane] + d.win_off;
  if (DIR == 0) block_copy<NT>(w, u, d.len); else block_copy<NT>(u, w, d.len);
}

// Uniform split with the header known on the host: a two-dimensional grid (tile in chunk, chunk)
// names the work directly, so a workgroup's only dependent access before its data is the one scalar
// load of its table row.
template <int DIR, int NT>
__global__ __launch_bounds__(kCopyBlock) void fl_copy_uniform(CopyArgs a) {
  warm_kernel_args(a);
  uint32_t bx = blockIdx.x, c = blockIdx.y;
  xcd_tile_2d(a.xcd, bx, c);
  if (c >= a.hint_n_chunks) return;
  const flh_chunk_desc d = a.table[c];
  const uint64_t off = (uint64_t)bx * a.tile_bytes;
  if (off >= d.len) return;
  const uint32_t bytes = (uint32_t)((d.len - off) < a.tile_bytes ? (d.len - off) : a.tile_bytes);
  bool ok = d.lane < a.win.n_lanes;
  if (ok) ok = d.win_off + d.len <= a.win.cap[d.lane] && d.src_off + d.len <= a.user_bytes;
  if (!ok) {
    if (threadIdx.x == 0) *a.status = FLH_E_RANGE;
    return;
  }
  uint8_t* u = a.user + d.src_off + off;
  uint8_t* w = (uint8_t*)a.win.base[d.lane] + d.win_off + off;
  if (DIR == 0) block_copy<NT>(w, u, bytes); else block_copy<NT>(u, w, bytes);
}

// Scheduler and copy in one launch, for the ordinary case of a uniform split under one credit row:
// the workgroup that copies tile k of chunk c works out the chunk's lane and window offset itself
// from the closed form (no table row to wait for), and the workgroup of tile 0 also writes the row
// out, so that the table exists for the receiver and for inspection exactly as the scheduler kernel
// would have produced it.  Window offsets start at zero (the windows are reused message by message).
struct FusedArgs {
  uint8_t* user;
  uint64_t user_bytes;
  flh_windows win;
  flh_chunk_desc* table;     // out (stripe only), may be null
  flh_sched_hdr* hdr;        // out (stripe only), may be null
  int32_t* status;
  uint64_t total_bytes;
  uint64_t src_base;
  uint64_t quanta_before;    // quanta of the current epoch already behind chunk 0 (epoch bytes / chunk)
  uint32_t chunk_bytes;
  uint32_t n_chunks;
  uint32_t n_lanes;
  uint32_t tile_bytes;
  uint32_t tiles_per_chunk;
  uint32_t dest_order;       // stripe only: blockIdx.y counts chunks in destination order (lane by lane)
  uint32_t credits[FLH_MAX_LANES];
  // Worked out once on the host when every quantum index and the credit sum W fit 32 bits: the per-workgroup
  // division by W becomes one multiply-high by magic = ceil(2^64 / W) (exact for 32-bit operands), and the
  // lane's slots before the message come from cnt0[] instead of a second and third division.
  // The lane of a slot is then found by a four-step binary search over pfx_ex[] (exclusive credit prefixes,
  // W from index n_lanes on), read straight from the argument block.
  uint32_t fast;
  uint32_t done_value;       // see done_word
  uint64_t magic;
  uint32_t cnt0[FLH_MAX_LANES];
  uint32_t pfx_ex[FLH_MAX_LANES + 1];
  uint32_t xcd_map;          // xcd_tile_2d()'s map for the grid (tiles per chunk, chunks); 0 = off
  // Reassembly only, may be null: a host-visible word that the last workgroup to finish sets to done_value, after
  // every workgroup's stores have been released (counted in *done_count, device memory, zero between launches).
  uint32_t* done_word;
  uint32_t* done_count;
  // Striping only, may be null: a host-visible word that the launch's first workgroup sets to start_value as it
  // starts.  A kernel starts once everything queued before it on its stream has finished, so a caller that numbers
  // its launches learns from the word that all earlier ones are complete.
  uint32_t* start_word;
  uint32_t start_value;
  uint32_t pad_start;
};

// Several requests in one launch.  Chunk c (counted over the launch) belongs to the request r with
// first[r] <= c < first[r + 1]; its bytes live at req_user[r] + (c - first[r]) * chunk_bytes.  Request r belongs to
// segment seg_of[r], and a segment is scheduled as the one message its requests form, from its own place in its credit
// epoch under its own credit row (the per-segment constants are those FusedArgs holds for a lone message), into the
// windows from base128[lane] * 128 on.
struct BatchSeg {
  uint64_t magic;                           // ceil(2^64 / W); 0 stands for W == 1
  uint32_t quanta_before;
  uint32_t first_chunk;
  uint32_t pfx_ex[FLH_MAX_LANES + 1];       // exclusive credit prefixes, W from index n_lanes on
  uint32_t cnt0[FLH_MAX_LANES];             // the lane's slots before the segment
  uint32_t base128[FLH_MAX_LANES];          // where the segment starts in the lane's window, in units of 128 bytes
  uint32_t n_chunks;
  uint32_t short_by;                        // bytes by which its last chunk falls short of chunk_bytes
  uint32_t zero;                            // the row had no credit (equal credits stand in)
  uint32_t pad;
};
struct FusedBatchArgs : FusedArgs {
  uint32_t n_req, n_seg;
  uint32_t first[FLH_BATCH_MAX];            // first chunk of each request; 0xffffffff from n_req on
  uint8_t seg_of[FLH_BATCH_MAX];
  uint8_t* req_user[FLH_BATCH_MAX];
  uint64_t req_bytes[FLH_BATCH_MAX];
  BatchSeg seg[FLH_SEG_MAX];
};
// Wire sends: a second set of windows, the receiver's landing windows.  The workgroup that has staged a tile in its
// lane's window then carries it into the same lane and offset of this set, the part the NIC of that lane plays in the
// reference (an RDMA write out of the staged copy, plugin.cc:1453-1495, 1582).  Argument blocks of their own, so that
// the launches without a wire keep theirs as they are.
// Where a staged tile goes next is either the same lane and offset of `carry` or, when `onward` names a buffer, the
// same place of that buffer as the tile has in its source: the receive buffer of a receiver whose memory this process
// can write (itself, or a process that exported the buffer), which is where the reference's RDMA write lands.
struct FusedCarryArgs : FusedArgs { flh_windows carry; uint8_t* onward; uint64_t onward_bytes; };
struct FusedBatchCarryArgs : FusedBatchArgs { flh_windows carry; uint8_t* onward[FLH_BATCH_MAX]; };   // one per request, or all null
static_assert(sizeof(FusedBatchCarryArgs) <= 4096, "a kernel's argument block holds 4 KiB");
template <class A> struct is_batch { static constexpr bool value = false; };
template <> struct is_batch<FusedBatchArgs> { static constexpr bool value = true; };
template <> struct is_batch<FusedBatchCarryArgs> { static constexpr bool value = true; };
template <class A> struct has_carry { static constexpr bool value = false; };
template <> struct has_carry<FusedCarryArgs> { static constexpr bool value = true; };
template <> struct has_carry<FusedBatchCarryArgs> { static constexpr bool value = true; };

// The message lives in pages of a pool: byte b of it is byte b mod page_bytes of pool page
// page_table[b / page_bytes].  `user` is the pool; a tile never straddles a page (tile_bytes divides page_bytes).
struct FusedPageArgs : FusedArgs {
  const uint32_t* page_table;
  uint64_t pool_pages;
  uint64_t n_pages;        // entries of page_table the message covers
  uint32_t page_bytes;
  int32_t page_shift;      // >= 0 when page_bytes is a power of two
};
template <class A> struct is_paged { static constexpr bool value = false; };
template <> struct is_paged<FusedPageArgs> { static constexpr bool value = true; };

struct FusedRow {  // inclusive credit prefixes of the one row (equal credits if it is empty)
  uint64_t pfx[FLH_MAX_LANES];
  uint64_t W;
  bool zero;
};

__device__ __forceinline__ void fused_row(const FusedArgs& a, FusedRow& r) {
  uint64_t run = 0;
#pragma unroll
  for (int l = 0; l < FLH_MAX_LANES; ++l) { if ((uint32_t)l < a.n_lanes) run += a.credits[l]; r.pfx[l] = run; }
  r.zero = run == 0;
  if (r.zero) {
#pragma unroll
    for (int l = 0; l < FLH_MAX_LANES; ++l) r.pfx[l] = (uint32_t)l < a.n_lanes ? l + 1 : a.n_lanes;
    run = a.n_lanes;
  }
  r.W = run;
}

// slots y < x that belong to the lane with prefix bounds [K, hi)
__device__ __forceinline__ uint64_t fused_cnt(uint64_t W, uint64_t K, uint64_t hi, uint64_t x) {
  const uint64_t c = hi - K;
  const uint64_t full = div_u64(x, W);
  const uint64_t rem = x - full * W;
  const uint64_t part = rem <= K ? 0 : (rem - K < c ? rem - K : c);
  return full * c + part;
}

// One workgroup's share of a fused launch: tile bx of the chunk that grid row by stands for (`span` neighbouring tiles
// of that chunk from bx on, for a caller that hands out larger shares).  DIR 0: user buffer -> staging window, 1: window
// -> user buffer, 2: staging window -> the same lane and offset of the carry windows (the wire), 3: user buffer -> staging
// window and, from the same registers, on to where the staged bytes go next: the same place of the arguments' onward
// buffer (the message's, or the request's in a batch) or, without one, the same lane and offset of the carry windows.
template <int DIR, int NT, class Args>
__device__ __forceinline__ void fused_tile(const Args& a, uint32_t bx, uint32_t by, uint32_t span = 1) {
  constexpr bool BATCH = is_batch<Args>::value;
  constexpr bool PAGED = is_paged<Args>::value;
  if (by >= a.n_chunks) return;
  uint32_t c = by, lane = 0;
  uint64_t before;
  // where the chunk's bytes live on the user side (the one buffer, or its request's), its length, its place in the
  // message for the table, and where its lane's window starts for it
  uint8_t* user = a.user;
  uint8_t* onward_user = nullptr;
  uint64_t user_off, user_bytes = a.user_bytes, src_off, win_base = 0;
  uint32_t len;
  if constexpr (BATCH) {
    static_assert(FLH_BATCH_MAX == 32, "the search below takes five steps");
    uint32_t r = a.first[16] <= c ? 16 : 0;     // entries from n_req on hold 0xffffffff
    if (a.first[r + 8] <= c) r += 8;
    if (a.first[r + 4] <= c) r += 4;
    if (a.first[r + 2] <= c) r += 2;
    if (a.first[r + 1] <= c) r += 1;
    const BatchSeg& g = a.seg[a.seg_of[r]];     // scalar loads from the argument block, register offsets
    const uint32_t in_seg = c - g.first_chunk;
    const uint32_t j = g.quanta_before + in_seg;
    const uint32_t full = g.magic ? (uint32_t)__umul64hi((uint64_t)j, g.magic) : j;
    const uint32_t slot = j - full * g.pfx_ex[FLH_MAX_LANES];
    static_assert(FLH_MAX_LANES == 16, "the search below takes four steps");
    if (g.pfx_ex[lane + 8] <= slot) lane += 8;
    if (g.pfx_ex[lane + 4] <= slot) lane += 4;
    if (g.pfx_ex[lane + 2] <= slot) lane += 2;
    if (g.pfx_ex[lane + 1] <= slot) lane += 1;
    const uint32_t K = g.pfx_ex[lane], hi = g.pfx_ex[lane + 1];
    before = (uint64_t)full * (hi - K) + (slot - K) - g.cnt0[lane];
    win_base = (uint64_t)g.base128[lane] * 128u;
    user = a.req_user[r];
    if constexpr (DIR == 3) onward_user = a.onward[r];
    user_bytes = a.req_bytes[r];
    user_off = (uint64_t)(c - a.first[r]) * a.chunk_bytes;
    const uint64_t rem = user_bytes - user_off;
    len = (uint32_t)(rem < a.chunk_bytes ? rem : a.chunk_bytes);
    src_off = (uint64_t)in_seg * a.chunk_bytes;
  } else {
    if (DIR != 1 && a.dest_order) {
      FusedRow r;
      fused_row(a, r);
      uint64_t K = 0, hi = r.pfx[0];
      // by = k-th chunk in destination order: find the lane whose group holds k, then invert the
      // closed form -- the j-th slot of a lane with credit c_l and first slot K_l is (j / c_l) * W + K_l + j mod c_l.
      const uint64_t x0 = a.quanta_before, x1 = a.quanta_before + a.n_chunks;
      const uint64_t f0 = div_u64(x0, r.W), f1 = div_u64(x1, r.W);
      const uint64_t r0 = x0 - f0 * r.W, r1 = x1 - f1 * r.W;
      uint64_t k = by, cnt0 = 0;
      bool found = false;
      uint64_t lo = 0;
#pragma unroll
      for (int l = 0; l < FLH_MAX_LANES; ++l) {
        const uint64_t up = r.pfx[l], cl = up - lo;
        const uint64_t p0 = r0 <= lo ? 0 : (r0 - lo < cl ? r0 - lo : cl);
        const uint64_t p1 = r1 <= lo ? 0 : (r1 - lo < cl ? r1 - lo : cl);
        const uint64_t c0 = f0 * cl + p0;             // slots of the lane before this message
        const uint64_t nl = f1 * cl + p1 - c0;        // chunks of this message on the lane
        if (!found && (uint32_t)l < a.n_lanes) {
          if (k < nl) { found = true; lane = l; K = lo; hi = up; cnt0 = c0; } else { k -= nl; }
        }
        lo = up;
      }
      const uint64_t cl = hi - K;
      const uint64_t ja = cnt0 + k;                   // index among all slots of the lane in this epoch
      const uint64_t rnd = div_u64(ja, cl);
      c = (uint32_t)(rnd * r.W + K + (ja - rnd * cl) - a.quanta_before);
      before = k;
    } else if (a.fast) {
      const uint32_t j = (uint32_t)a.quanta_before + c;
      const uint32_t full = a.magic ? (uint32_t)__umul64hi((uint64_t)j, a.magic) : j;  // j / W (magic 0 stands for W = 1)
      const uint32_t slot = j - full * a.pfx_ex[FLH_MAX_LANES];  // the last entry is always W
      // the last lane whose first slot is not beyond this one (lanes without credit share their successor's first slot)
      static_assert(FLH_MAX_LANES == 16, "the search below takes four steps");
      if (a.pfx_ex[lane + 8] <= slot) lane += 8;
      if (a.pfx_ex[lane + 4] <= slot) lane += 4;
      if (a.pfx_ex[lane + 2] <= slot) lane += 2;
      if (a.pfx_ex[lane + 1] <= slot) lane += 1;
      const uint32_t K = a.pfx_ex[lane], hi = a.pfx_ex[lane + 1], c0 = a.cnt0[lane];   // indexed scalar loads from the argument block
      before = (uint64_t)full * (hi - K) + (slot - K) - c0;  // slot lies inside the lane's span [K, hi)
    } else {
      FusedRow r;
      fused_row(a, r);
      uint64_t K = 0, hi = r.pfx[0];
      const uint64_t j = a.quanta_before + c;
      const uint64_t slot = mod_u64(j, r.W);
#pragma unroll
      for (int l = 0; l + 1 < FLH_MAX_LANES; ++l) {
        if ((uint32_t)(l + 1) < a.n_lanes && r.pfx[l] <= slot) { lane = l + 1; K = r.pfx[l]; hi = r.pfx[l + 1]; }
      }
      before = fused_cnt(r.W, K, hi, j) - fused_cnt(r.W, K, hi, a.quanta_before);
    }
    const uint64_t chunk_off = (uint64_t)c * a.chunk_bytes;
    const uint64_t rem = a.total_bytes - chunk_off;
    len = (uint32_t)(rem < a.chunk_bytes ? rem : a.chunk_bytes);
    src_off = a.src_base + chunk_off;
    user_off = src_off;
    if constexpr (DIR == 3) {
      onward_user = a.onward;
      if (onward_user && user_off + len > a.onward_bytes) {
        if (bx == 0 && threadIdx.x == 0) st_obj<NT>(a.status, (int32_t)FLH_E_RANGE);
        return;
      }
    }
  }
  const uint64_t win_off = win_base + before * a.chunk_bytes;

  if ((DIR == 0 || DIR == 3) && bx == 0 && threadIdx.x == 0 && a.table) {
    flh_chunk_desc d;
    d.src_off = src_off;
    d.win_off = win_off;
    d.len = len;
    d.lane = lane;
    d.tile_base = c * a.tiles_per_chunk;
    d.epoch = 0;
    st_obj<NT>(&a.table[c], d);
  }
  if ((DIR == 0 || DIR == 3) && bx == 0 && by == 0 && a.hdr) {  // header: per-lane totals in closed form
    const uint32_t t = threadIdx.x;
    if constexpr (BATCH) {
      // the launch's totals: every segment's closed form, summed
      if (t < FLH_MAX_LANES) {
        uint64_t chunks = 0, bytes = 0;
        if (t < a.n_lanes) {
          for (uint32_t s = 0; s < a.n_seg; ++s) {
            const BatchSeg& g = a.seg[s];
            const uint32_t W = g.pfx_ex[FLH_MAX_LANES], K = g.pfx_ex[t], cl = g.pfx_ex[t + 1] - K;
            const uint32_t x1 = g.quanta_before + g.n_chunks;
            const uint32_t full = g.magic ? (uint32_t)__umul64hi((uint64_t)x1, g.magic) : x1;
            const uint32_t rem = x1 - full * W;
            const uint32_t part = rem <= K ? 0 : (rem - K < cl ? rem - K : cl);
            const uint64_t k = (uint64_t)full * cl + part - g.cnt0[t];
            const uint32_t xl = x1 - 1;                       // the segment's last chunk: short, and on which lane
            const uint32_t fl = g.magic ? (uint32_t)__umul64hi((uint64_t)xl, g.magic) : xl;
            const uint32_t sl = xl - fl * W;
            chunks += k;
            bytes += k * a.chunk_bytes - ((g.n_chunks && sl >= K && sl < K + cl) ? g.short_by : 0);
          }
        }
        st_obj<NT>(&a.hdr->lane_bytes[t], bytes);
        st_obj<NT>(&a.hdr->lane_chunks[t], (uint32_t)chunks);
      }
      if (t == 0) {
        uint32_t tiles = 0, zero = 0;
        for (uint32_t s = 0; s < a.n_seg; ++s) {
          const BatchSeg& g = a.seg[s];
          if (!g.n_chunks) continue;
          tiles += (g.n_chunks - 1) * a.tiles_per_chunk + (a.chunk_bytes - g.short_by + a.tile_bytes - 1) / a.tile_bytes;
          zero |= g.zero;
        }
        st_obj<NT>(&a.hdr->total_bytes, a.total_bytes);
        st_obj<NT>(&a.hdr->total_tiles, tiles);
        st_obj<NT>(&a.hdr->n_chunks, a.n_chunks);
        st_obj<NT>(&a.hdr->flags, (uint32_t)(zero ? FLH_SCHED_F_NO_CREDIT : 0));
        st_obj<NT>(&a.hdr->uniform_tiles, a.tiles_per_chunk);
      }
    } else {
      FusedRow r;
      fused_row(a, r);
      const uint64_t last = a.n_chunks - 1;
      const uint64_t len_last = a.total_bytes - last * a.chunk_bytes;
      if (t < FLH_MAX_LANES) {
        uint64_t chunks = 0, bytes = 0;
        if (t < a.n_lanes) {
          uint64_t k_lo = 0, k_hi = 0;  // selected, not indexed: indexing would push the row into scratch memory
#pragma unroll
          for (int l = 0; l < FLH_MAX_LANES; ++l) {
            if ((uint32_t)l == t) { k_hi = r.pfx[l]; k_lo = l ? r.pfx[l > 0 ? l - 1 : 0] : 0; }
          }
          chunks = fused_cnt(r.W, k_lo, k_hi, a.quanta_before + a.n_chunks) - fused_cnt(r.W, k_lo, k_hi, a.quanta_before);
          const uint64_t slot_last = mod_u64(a.quanta_before + last, r.W);
          const bool mine = slot_last >= k_lo && slot_last < k_hi;
          bytes = chunks * a.chunk_bytes - (mine ? a.chunk_bytes - len_last : 0);
        }
        st_obj<NT>(&a.hdr->lane_bytes[t], bytes);
        st_obj<NT>(&a.hdr->lane_chunks[t], (uint32_t)chunks);
      }
      if (t == 0) {
        st_obj<NT>(&a.hdr->total_bytes, a.total_bytes);
        st_obj<NT>(&a.hdr->total_tiles, (uint32_t)last * a.tiles_per_chunk + (uint32_t)((len_last + a.tile_bytes - 1) / a.tile_bytes));
        st_obj<NT>(&a.hdr->n_chunks, a.n_chunks);
        st_obj<NT>(&a.hdr->flags, (uint32_t)(r.zero ? FLH_SCHED_F_NO_CREDIT : 0));
        st_obj<NT>(&a.hdr->uniform_tiles, a.tiles_per_chunk);
      }
    }
  }

  const uint64_t off = (uint64_t)bx * a.tile_bytes;
  if (off >= len) return;
  const uint64_t share = (uint64_t)a.tile_bytes * span;
  const uint32_t bytes = (uint32_t)((len - off) < share ? (len - off) : share);
  if (win_off + len > a.win.cap[lane] || (!PAGED && user_off + len > user_bytes)) {
    if (threadIdx.x == 0) st_obj<NT>(a.status, (int32_t)FLH_E_RANGE);
    return;
  }
  uint8_t* u = user + user_off + off;
  if constexpr (PAGED) {
    const uint64_t at = src_off + off;   // the tile's first byte in the message
    const uint64_t pi = a.page_shift >= 0 ? at >> a.page_shift : at / a.page_bytes;
    const uint32_t pg = pi < a.n_pages ? a.page_table[pi] : 0xffffffffu;
    if (pg >= a.pool_pages) {
      if (threadIdx.x == 0) st_obj<NT>(a.status, (int32_t)FLH_E_RANGE);
      return;
    }
    u = user + (uint64_t)pg * a.page_bytes + (at - pi * a.page_bytes);
  }
  uint8_t* w = (uint8_t*)a.win.base[lane] + win_off + off;
  if constexpr (DIR == 2) {
    static_assert(has_carry<Args>::value, "the carry needs landing windows");
    if (win_off + len > a.carry.cap[lane]) {
      if (threadIdx.x == 0) st_obj<NT>(a.status, (int32_t)FLH_E_RANGE);
      return;
    }
    block_copy<NT>((uint8_t*)a.carry.base[lane] + win_off + off, w, bytes);
  } else if constexpr (DIR == 3) {
    static_assert(has_carry<Args>::value && !PAGED, "the second destination is a receive buffer or a landing window");
    // bit 4 of the mode: the window's stores stream (bit 1 speaks for the stores that go on)
    constexpr int NTW = (NT & ~(2 | 16)) | ((NT & 16) ? 2 : 0), NTO = NT & ~16;
    if (onward_user) {
      block_copy2<NTW, NTO>(w, onward_user + user_off + off, u, bytes);
    } else {
      if (win_off + len > a.carry.cap[lane]) {   // refused whole: nothing of the chunk is staged either
        if (threadIdx.x == 0) st_obj<NT>(a.status, (int32_t)FLH_E_RANGE);
        return;
      }
      block_copy2<NTW, NTO>(w, (uint8_t*)a.carry.base[lane] + win_off + off, u, bytes);
    }
  } else if constexpr (DIR == 0) {
    block_copy<NT>(w, u, bytes);
  } else {
    block_copy<NT>(u, w, bytes);
  }
}

template <int DIR, int NT, class Args>
__global__ __launch_bounds__(kCopyBlock) void fl_copy_uniform_fused(Args a) {
  warm_kernel_args(a);
  uint32_t bx = blockIdx.x, by = blockIdx.y;   // tile of the chunk, chunk (in message or destination order)
  xcd_tile_2d(a.xcd_map, bx, by);
  if (a.start_word && bx == 0 && by == 0 && threadIdx.x == 0)
    __hip_atomic_store(a.start_word, a.start_value, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
  // with a wire: the tile goes into its staging window and, from the same registers, into the landing windows
  if constexpr (DIR == 0 && has_carry<Args>::value) fused_tile<3, NT>(a, bx, by);
  else fused_tile<DIR, NT>(a, bx, by);
  // Completion word.  Every workgroup of the grid comes through here, also those without a tile.  The barrier orders
  // the workgroup's stores before thread 0's increment, which releases them at agent scope; the workgroup that counts
  // the last one has thereby acquired every other workgroup's stores, and its store of the word releases all of them
  // at system scope.  A reader that finds done_value with an acquire load may read the destination.
  if ((DIR == 1 || has_carry<Args>::value) && a.done_word) {
    __syncthreads();
    if (threadIdx.x == 0) {
      const uint32_t total = gridDim.x * gridDim.y;
      const uint32_t prev = __hip_atomic_fetch_add(a.done_count, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
      if (prev + 1 == total) {
        __hip_atomic_store(a.done_count, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(a.done_word, a.done_value, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
      }
    }
  }
}

struct PageArgs {
  uint8_t* pool;
  uint64_t pool_pages;
  const uint32_t* page_table;
  flh_windows win;
  const flh_chunk_desc* table;
  int32_t* status;
  uint32_t n_chunks;
  uint32_t page_bytes;
  uint32_t pages_per_chunk;
  uint32_t sub_bytes;      // bytes of a page handled by one workgroup step
  uint32_t subs_per_page;
  int32_t page_shift;      // >= 0 when page_bytes is a power of two
  uint32_t xcd_map;        // xcd_tile_2d()'s map when the grid has one row per chunk; 0 = off
};

constexpr uint32_t kLdsStage = 16384;

// DIR 0: pool pages -> windows (gather).  DIR 1: windows -> pool pages (scatter).
// LDS: stage each sub-tile through LDS (coalesced global->LDS, barrier, LDS->global).
template <int DIR, int NT, bool LDS>
__global__ __launch_bounds__(kCopyBlock) void fl_page_tiles(PageArgs a) {
  __shared__ u32x4 stage[LDS ? kLdsStage / 16 : 1];
  warm_kernel_args(a);
  // grid: x = (page in chunk, part of page), y = chunk (stepping by the grid's height past 65535 chunks); no
  // 64-bit division stands between a workgroup and its row
  uint32_t bx = blockIdx.x, by = blockIdx.y;
  xcd_tile_2d(a.xcd_map, bx, by);
  const uint32_t k = a.subs_per_page == 1 ? bx : bx / a.subs_per_page;
  const uint32_t sub = bx - k * a.subs_per_page;
  for (uint32_t c = by; c < a.n_chunks; c += gridDim.y) {
    const flh_chunk_desc d = a.table[c];
    const uint64_t in_chunk = (uint64_t)k * a.page_bytes + (uint64_t)sub * a.sub_bytes;
    if (in_chunk >= d.len) continue;
    uint32_t bytes = a.page_bytes - sub * a.sub_bytes;
    if (bytes > a.sub_bytes) bytes = a.sub_bytes;
    if (bytes > d.len - in_chunk) bytes = (uint32_t)(d.len - in_chunk);
    // the chunk's place in the message comes from its source offset, not from the row's position, so the
    // rows may come in any order (destination order for the gather)
    const uint64_t p = (a.page_shift >= 0 ? d.src_off >> a.page_shift : d.src_off / a.page_bytes) + k;
    const bool aligned = a.page_shift >= 0 ? (d.src_off & (a.page_bytes - 1)) == 0 : d.src_off % a.page_bytes == 0;
    if (!aligned || p >= (uint64_t)a.n_chunks * a.pages_per_chunk) {
      if (threadIdx.x == 0) *a.status = FLH_E_RANGE;
      continue;
    }
    const uint32_t pg = a.page_table[p];
    bool ok = d.lane < a.win.n_lanes && pg < a.pool_pages;
    if (ok) ok = d.win_off + d.len <= a.win.cap[d.lane];
    if (!ok) {
      if (threadIdx.x == 0) *a.status = FLH_E_RANGE;
      continue;
    }
    uint8_t* u = a.pool + (uint64_t)pg * a.page_bytes + (uint64_t)sub * a.sub_bytes;
    uint8_t* w = (uint8_t*)a.win.base[d.lane] + d.win_off + in_chunk;
    uint8_t* dst = DIR == 0 ? w : u;
    const uint8_t* src = DIR == 0 ? u : w;
    if (LDS && ((((uintptr_t)src | (uintptr_t)dst) & 15) == 0) && (bytes & 15) == 0) {
      const uint32_t nvec = bytes >> 4;  // <= kLdsStage/16 by construction of sub_bytes
      const u32x4* s = (const u32x4*)src;
      u32x4* dd = (u32x4*)dst;
      for (uint32_t i = threadIdx.x; i < nvec; i += kCopyBlock) stage[i] = ld16<NT>(s + i);
      __syncthreads();
      for (uint32_t i = threadIdx.x; i < nvec; i += kCopyBlock) st16<NT>(dd + i, stage[i]);
      __syncthreads();
    } else {
      block_copy<NT>(dst, src, bytes);
    }
  }
}

template <int NT>
__global__ __launch_bounds__(kCopyBlock) void fl_plain_copy(uint8_t* dst, const uint8_t* src, uint64_t bytes,
                                                            uint32_t tile_bytes, uint32_t xcd) {
  const uint64_t tiles = (bytes + tile_bytes - 1) / tile_bytes;
  for (uint64_t t = xcd_tile(blockIdx.x, xcd); t < tiles; t += gridDim.x) {
    const uint64_t off = t * tile_bytes;
    const uint32_t len = (uint32_t)((bytes - off) < tile_bytes ? (bytes - off) : tile_bytes);
    block_copy<NT>(dst + off, src + off, len);
  }
}

// Up to FLH_MAX_LANES independent runs in one launch (flh_copy_runs): a workgroup per copy tile, the run of a tile
// found by a four-step search over the runs' first tiles in the argument block.
struct CopyRuns {
  uint8_t* dst[FLH_MAX_LANES];
  const uint8_t* src[FLH_MAX_LANES];
  uint64_t bytes[FLH_MAX_LANES];
  uint32_t first_tile[FLH_MAX_LANES + 1];   // exclusive prefix of the runs' tile counts; entries past the last run repeat the total
  uint32_t tile_bytes;
  uint32_t xcd;
};

template <int NT>
__global__ __launch_bounds__(kCopyBlock) void fl_copy_runs(CopyRuns a) {
  warm_kernel_args(a);
  const uint32_t t = (uint32_t)xcd_tile(blockIdx.x, a.xcd);
  static_assert(FLH_MAX_LANES == 16, "the search below takes four steps");
  uint32_t r = 0;
  if (a.first_tile[r + 8] <= t) r += 8;
  if (a.first_tile[r + 4] <= t) r += 4;
  if (a.first_tile[r + 2] <= t) r += 2;
  if (a.first_tile[r + 1] <= t) r += 1;
  const uint64_t off = (uint64_t)(t - a.first_tile[r]) * a.tile_bytes;
  const uint64_t n = a.bytes[r];
  if (off >= n) return;
  const uint32_t len = (uint32_t)((n - off) < a.tile_bytes ? (n - off) : a.tile_bytes);
  block_copy<NT>(a.dst[r] + off, a.src[r] + off, len);
}

// ------------------------------------------------------------------------------------------------
// lane engine: a resident kernel that executes batch descriptors
// ------------------------------------------------------------------------------------------------
// Launching a stripe + reassemble pair costs the host about ten microseconds, which bounds the request rate at NCCL's
// 512 KiB steps.  The engine takes the launches off that path: the host writes the descriptor of a batch -- the very
// argument block the batch kernels take -- into a ring in pinned memory and advances a tail word; one workgroup of the
// resident kernel (the dispatcher) polls the tail, copies new descriptors into device memory and publishes them, and
// the other workgroups (the workers) run every batch's tiles through the same routine the launched kernels run
// (fused_tile): a tile is loaded once and stored twice, into its lane's staging window and on to where the staged bytes
// go next (the receive buffer, or the receiving process's landing window), so no workgroup waits for another inside
// a batch and nothing is read back.  A batch's tiles go to the
// workers in turn, starting behind the worker that took the last tile of the batch before, so that small batches
// run side by side on different workers.  Only the workers with a share in a batch are counted in and out of it: the
// others pass it by without an atomic, so what a small batch costs does not grow with the size of the engine.  The
// workers never reach a kernel boundary, which is where a kernel's view of memory is brought up to date and its stores
// are made visible; they touch memory at system scope instead (streaming modes 4 and 8 of the copies) and so need no
// cache invalidate or L2 write-back per batch.  Successive batches rotate through the caller's sets of staging windows,
// and a worker enters batch k only once batch k - sets is complete.  The last worker to leave a batch stores its number to a host-visible word of the
// batch's ring slot; batches of different workers may complete out of order, and the host reports the complete prefix.
// Every wait in the kernel is bounded: with nothing to do for idle_us the dispatcher takes the engine down (the host
// starts it again with the next batch), and a wait that outlasts wait_us reports an error and takes it down as well.
constexpr uint32_t kEngineDevRing = 8;          // descriptors held in device memory; also the most window sets a caller may rotate
constexpr uint32_t kEngineDescBytes = 4096;
// A worker takes one copy tile at a time (32 KiB) from a batch that then still leaves a quarter of the workers to the
// batches beside it, and two neighbouring tiles (64 KiB, what a workgroup has in flight when every thread issues its
// sixteen loads at once) from a larger one.  Shares of one tile are latency: a batch of one or four 512 KiB requests on
// its own takes 10.0 / 10.3 us instead of 12.1, four such in flight are served as fast either way (3.5-3.6 us each).
// Shares of two are throughput: with one-tile shares a batch of eight spreads over all 128 workers and four in flight
// are served every 6.1 instead of every 4.1 us.  Under the plugin (batches of three to five requests) a limit of 64, 96,
// 128 tiles or none gave the same rates within the spread of three runs each, all of them above two-tile shares
// throughout (one connection 849 against 886-971 GB/s, four 1 980 against 2 083-2 122).
constexpr uint32_t kEngineShareMax = 2;
inline uint32_t engine_share(uint32_t batch_tiles, uint32_t workers) {
  const uint64_t upto = g_lane_share1_tiles < 0 ? (uint64_t)workers * 3 / 4 : (uint64_t)g_lane_share1_tiles;   // flh_tune("lane_share1_tiles")
  return batch_tiles <= upto ? 1u : kEngineShareMax;
}

// What a batch does with its tiles.  Loop: user buffers -> staging windows -> receive buffers, both ends in this process.
// Send: user buffers -> staging windows -> the same lane and offset of the landing windows (FusedArgs::carry), which are
// the receiving process's memory: staging plus the wire.  Receive: landing windows (given as the batch's windows) ->
// receive buffers.
enum : uint32_t { kEngineLoop = FLH_ENGINE_LOOP, kEngineSend = FLH_ENGINE_SEND, kEngineRecv = FLH_ENGINE_RECV };
struct EngineDesc {                              // what the host writes per batch (kEngineDescBytes at most)
  uint32_t tiles;                                // worker shares of the batch (the slot's first word: the dispatcher's thread 0 has it in hand)
  uint32_t kind;
  uint32_t share;                                // copy tiles per share (engine_share)
  uint32_t pad;
  FusedBatchCarryArgs a;                         // as the striping launch would take it (req_user = sources, onward = the receive buffers of a kEngineLoop batch; kEngineRecv: req_user = the receive buffers)
};
static_assert(sizeof(EngineDesc) <= kEngineDescBytes, "descriptor slot too small");

struct EngineHostCtl {                           // pinned host memory, mapped to the device; one 64-byte line per word
  alignas(64) uint64_t tail;                     // host: batches submitted so far
  alignas(64) uint32_t state;                    // 0 down, 1 running, 2 about to go down (device; the host sets 1 when it launches)
  alignas(64) uint64_t exited_at;                // device: the batch the next engine has to start with
  alignas(64) uint64_t done[kEngineDevRing];     // device: per ring slot, the number of the last batch of that slot that is complete
  alignas(64) int32_t error;                     // device: a bounded wait ran out (FLH_E_STATE)
  alignas(64) uint32_t stop;                     // host: go down now
};
struct EngineDevCtl {                            // device memory
  // per ring slot, one word from which a worker learns that its batch is there, which of its shares (if any) are its
  // own, when it may enter and whether it is the last to leave (engine_word): the batch's number, the worker that
  // takes its first share, its shares, and the slot counters' values that mean "this batch is complete" and "the batch
  // whose windows it reuses is complete"
  alignas(64) uint64_t published[kEngineDevRing];
  alignas(64) uint32_t quit;                     // the engine launch (EngineArgs::gen) whose workers leave when they reach batch quit_at; never cleared
  uint32_t pad;
  uint64_t quit_at;
  alignas(64) uint64_t arrive[kEngineDevRing];   // workers with a share that have left the batches of each ring slot, never reset
  alignas(64) uint64_t target[kEngineDevRing];   // the dispatcher's record: arrive[slot] once the slot's latest batch is complete (kept across engine launches)
  // per ring slot, the number of the last batch of the slot whose completion word has reached the host (stored by the
  // worker that stored the word, once that store has been acknowledged).  The dispatcher gives a slot to batch k only
  // once this says k - ring: the completion word of a slot can then never be stored out of order, however long the
  // last worker of a batch dawdles between counting itself out and storing the word.
  alignas(64) uint64_t freed[kEngineDevRing];
};

// The published word: batch number (16 bits) | first worker (10) | shares, saturated (10) | low 14 bits of the slot
// counter when this batch is complete | low 14 bits of the counter of slot (k - sets) when that batch is complete.
// Counters are compared modulo 2^14: a slot's counter is never more than one batch (at most 1023 workers) away from
// either value while anyone looks.
constexpr uint32_t kEngineCountMask = 0x3fffu;
__host__ __device__ inline uint64_t engine_word(uint64_t k, uint32_t first, uint32_t shares, uint64_t own_target, uint64_t wait_target) {
  return ((uint64_t)(uint16_t)(k + 1) << 48) | ((uint64_t)(first & 0x3ffu) << 38) | ((uint64_t)(shares < 0x3ffu ? shares : 0x3ffu) << 28) |
         ((own_target & kEngineCountMask) << 14) | (wait_target & kEngineCountMask);
}
struct EngineArgs {
  const uint8_t* host_ring;                      // kHostRing descriptors, device-visible pinned memory
  uint32_t host_slots;
  uint32_t workers;
  uint32_t sets;                                 // the caller rotates this many window sets: batch k waits for batch k - sets
  uint32_t gen;                                  // number of this launch of the engine, from 1: what the quit word must hold to mean this one
  EngineHostCtl* hctl;
  uint8_t* dev_ring;
  EngineDevCtl* dctl;
  uint64_t start;                                // first batch to execute
  uint64_t idle_ticks, wait_ticks;               // of the 100 MHz wall clock
  uint64_t resident_ticks;                       // the engine leaves after this long even with work at hand (0: never); the host starts it again
  uint32_t inject_fault;                         // tests of the failure path: fail in place of executing the first batch
  uint32_t trace_mask;                           // trace slots - 1 (a power of two of them)
  uint64_t* trace;                               // null, or kEngineStamps wall-clock stamps per slot: where a batch's time goes (flh_engine_trace)
};

// Stamps of one batch (100 MHz wall clock): the dispatcher has seen the host's tail beyond it; has published it; the
// worker with its first share has seen the published word; may enter (the batch whose windows it reuses is complete);
// has the descriptor in LDS; has moved its shares and its stores are in memory; the last worker out has the completion
// word's store acknowledged.
enum : uint32_t { kStampTail, kStampPublished, kStampSeen, kStampEntered, kStampDesc, kStampMoved, kStampDone, kEngineStamps };
static_assert(kEngineStamps == FLH_ENGINE_STAMPS, "the header's count of stamps");
__device__ __forceinline__ void engine_stamp(const EngineArgs& e, uint64_t k, uint32_t what) {
  if (e.trace) __hip_atomic_store(&e.trace[(k & e.trace_mask) * kEngineStamps + what], wall_clock64(), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

__device__ __forceinline__ void engine_fail(const EngineArgs& e) {
  __hip_atomic_store(&e.hctl->error, (int32_t)FLH_E_STATE, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  __hip_atomic_store(&e.dctl->quit_at, (uint64_t)0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __hip_atomic_store(&e.dctl->quit, e.gen, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
}

__global__ __launch_bounds__(kCopyBlock) void fl_engine_kernel(EngineArgs e) {
  __shared__ EngineDesc d;
  __shared__ uint32_t sh_flag, sh_first;
  __shared__ uint64_t sh_word;
  __shared__ uint64_t tgt[kEngineDevRing];
  const uint32_t tid = threadIdx.x;
  const uint32_t W = e.workers;
  if (blockIdx.x == 0) {
    // ---- dispatcher ------------------------------------------------------------------------------------------
    uint64_t k = e.start;
    uint64_t tail_seen = e.start;   // the host's tail as last read: a burst of batches costs one look across the bus
    uint32_t first_worker = 0;      // takes the first tile of batch k
    uint32_t polls = 0;
    uint64_t idle_since = wall_clock64(), free_since = idle_since;
    const uint64_t born = idle_since;
    if (tid < kEngineDevRing) tgt[tid] = e.dctl->target[tid];   // where the engine before this one left the slots
    __syncthreads();
    for (;;) {
      if (tid == 0) {
        uint32_t act = 0;   // 0 poll again, 1 copy descriptor k, 2 leave
        const uint64_t now = wall_clock64();
        if (e.resident_ticks && now - born > e.resident_ticks) {
          // Resident long enough.  A kernel that never ends holds its hardware queue, and whatever the runtime has
          // put on the same queue behind it (streams outnumber queues) waits for as long as small requests keep
          // coming.  So the engine leaves between two batches although there may be work, and the host starts the
          // next one (the submit that finds the state at 0, or flh_engine_poke): the queue drains in between.
          __hip_atomic_store(&e.hctl->state, 2u, __ATOMIC_SEQ_CST, __HIP_MEMORY_SCOPE_SYSTEM);
          act = 2;
        } else
        // the device slot of batch k held batch k - ring: that one must be complete and its completion word out
        if (__hip_atomic_load(&e.dctl->arrive[k % kEngineDevRing], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >= tgt[k % kEngineDevRing] &&
            (k < kEngineDevRing || __hip_atomic_load(&e.dctl->freed[k % kEngineDevRing], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + kEngineDevRing >= k + 1)) {
          free_since = now;
          if (tail_seen <= k) tail_seen = __hip_atomic_load(&e.hctl->tail, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_SYSTEM);
          if (tail_seen > k) act = 1;
        } else if (now - free_since > e.wait_ticks) {
          engine_fail(e);   // the workers never left the batch that holds the slot
        }
        if (act == 1 && e.inject_fault) {
          engine_fail(e);   // as if a wait had run out: the batch stays unexecuted, everybody leaves
          act = 2;
        }
        if (act == 1) {
          idle_since = now;
          engine_stamp(e, k, kStampTail);
          __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");   // the workers' reads of the slot are behind their arrival
        } else if (__hip_atomic_load(&e.dctl->quit, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == e.gen ||
                   ((++polls & 31) == 0 && __hip_atomic_load(&e.hctl->stop, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM))) {
          act = 2;   // (the host's stop flag is a trip across the bus: looked at now and then)
        } else if (now - idle_since > e.idle_ticks) {
          // Nothing for a while: announce it, then look once more.  The host stores the tail, then reads the state; this
          // side stores the state, then reads the tail: one of the two sees the other's store.
          __hip_atomic_store(&e.hctl->state, 2u, __ATOMIC_SEQ_CST, __HIP_MEMORY_SCOPE_SYSTEM);
          __atomic_thread_fence(__ATOMIC_SEQ_CST);
          const uint64_t tail = __hip_atomic_load(&e.hctl->tail, __ATOMIC_SEQ_CST, __HIP_MEMORY_SCOPE_SYSTEM);
          if (tail > k) {
            __hip_atomic_store(&e.hctl->state, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
            idle_since = now;
          } else {
            act = 2;
          }
        }
        sh_flag = act;
      }
      __syncthreads();
      const uint32_t act = sh_flag;
      __syncthreads();
      if (act == 2) break;
      if (act == 0) { __builtin_amdgcn_s_sleep(2); continue; }
      // descriptor k: pinned host memory -> device ring, sixteen bytes per thread
      const u32x4* src = (const u32x4*)(e.host_ring + (size_t)(k % e.host_slots) * kEngineDescBytes);
      u32x4* dst = (u32x4*)(e.dev_ring + (size_t)(k % kEngineDevRing) * kEngineDescBytes);
      static_assert(kEngineDescBytes == kCopyBlock * 16, "one vector per thread moves a descriptor");
      const u32x4 v = src[tid];
      dst[tid] = v;
      __syncthreads();
      if (tid == 0) {
        const uint32_t tiles = v.x;                                 // EngineDesc::tiles: the batch's shares
        const uint32_t slot = (uint32_t)(k % kEngineDevRing);
        const uint64_t takers = tiles < W ? tiles : W;              // workers with a share in the batch
        const uint64_t wait_target = k >= e.sets ? tgt[(k - e.sets) % kEngineDevRing] : 0;   // (read before this slot's own entry moves: sets may equal the ring)
        const uint64_t own_target = tgt[slot] + takers;
        tgt[slot] = own_target;
        e.dctl->target[slot] = own_target;
        __hip_atomic_store(&e.dctl->published[slot], engine_word(k, first_worker, tiles, own_target, wait_target), __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
        engine_stamp(e, k, kStampPublished);
        if (takers == 0) {   // nothing to move (the host submits no such batch): complete as it stands
          __hip_atomic_store(&e.hctl->done[slot], k + 1, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
          asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
          __hip_atomic_store(&e.dctl->freed[slot], k + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        first_worker = (uint32_t)((first_worker + tiles) % W);
      }
      ++k;
    }
    if (tid == 0) {
      // workers finish what has been published and leave at batch k; the next engine starts there
      if (__hip_atomic_load(&e.dctl->quit, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != e.gen) {
        __hip_atomic_store(&e.dctl->quit_at, k, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(&e.dctl->quit, e.gen, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
      }
      __hip_atomic_store(&e.hctl->exited_at, k, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
      __hip_atomic_store(&e.hctl->state, 0u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
    }
    return;
  }
  // ---- worker ----------------------------------------------------------------------------------------------
  const uint32_t w = blockIdx.x - 1;
  for (uint64_t k = e.start;; ++k) {
    if (tid == 0) {
      uint32_t act = 1;   // 1 run batch k, 2 leave, 3 no share of batch k is this worker's
      uint64_t word = 0;
      const uint64_t t0 = wall_clock64();
      for (uint32_t spin = 0;; ++spin) {
        word = __hip_atomic_load(&e.dctl->published[k % kEngineDevRing], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // (what it announces is then loaded at system scope)
        const int16_t ahead = (int16_t)((uint16_t)(word >> 48) - (uint16_t)(k + 1));
        if (ahead == 0) break;
        // the slot already holds a later batch: batch k came and went, which it could not have with a share of this worker outstanding
        if (ahead > 0) { act = 3; break; }
        if ((spin & 7) == 7) {   // the flag and the clock now and then: every look is a round trip to memory
          if (__hip_atomic_load(&e.dctl->quit, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == e.gen &&
              __hip_atomic_load(&e.dctl->quit_at, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) <= k) { act = 2; break; }
          if (wall_clock64() - t0 > e.wait_ticks + e.idle_ticks) { engine_fail(e); act = 2; break; }
        }
        __builtin_amdgcn_s_sleep(1);
      }
      // this worker's first share of the batch: the shares go round the workers from the batch's first worker on
      const uint32_t first = (uint32_t)(word >> 38) & 0x3ffu;
      sh_first = (w + W - first) % W;
      if (act == 1 && sh_first >= ((uint32_t)(word >> 28) & 0x3ffu)) act = 3;
      if (act == 1 && sh_first == 0) engine_stamp(e, k, kStampSeen);
      if (act == 1 && k >= e.sets) {
        // batch k reuses the windows of batch k - sets: that one must be complete
        const uint64_t j = k - e.sets;
        const uint32_t need = (uint32_t)word & kEngineCountMask;
        const uint64_t t1 = wall_clock64();
        while ((((uint32_t)__hip_atomic_load(&e.dctl->arrive[j % kEngineDevRing], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) - need) & kEngineCountMask) > kEngineCountMask / 2) {
          if (wall_clock64() - t1 > e.wait_ticks) { engine_fail(e); act = 2; break; }
          __builtin_amdgcn_s_sleep(1);
        }
      }
      if (act == 1 && sh_first == 0) engine_stamp(e, k, kStampEntered);
      sh_flag = act;
      sh_word = word;
    }
    __syncthreads();
    const uint32_t act = sh_flag, mine = sh_first;
    const uint32_t own_target = (uint32_t)(sh_word >> 14) & kEngineCountMask;
    __syncthreads();
    if (act == 2) return;
    if (act == 3) continue;   // nothing read, nothing written, nothing to count
    uint64_t* cnt = &e.dctl->arrive[k % kEngineDevRing];
    // What the batch reads may have been written by anyone, on this GPU or off it, before the host submitted it, and
    // what it writes is read by anyone once the host has seen it complete.  A worker therefore loads the descriptor and
    // the sources at system scope (mode 8: from memory, whatever line a cache has kept) and stores at system scope
    // (mode 4: written through).  So it needs no cache invalidate on its way into a batch and no L2 write-back on its
    // way out.
    // Either of the two costs every workgroup that shares the XCD's L2: with 64 workers per batch fencing, batches of
    // eight 512 KiB requests were served every 7.4 us, now every 3.8 us.
    {
      const VecIn<8> slot((const u32x4*)(e.dev_ring + (size_t)(k % kEngineDevRing) * kEngineDescBytes), kEngineDescBytes / 16);
      u32x4* dst = (u32x4*)&d;
      if (tid * 16 < sizeof(EngineDesc)) dst[tid] = slot(tid);
    }
    __syncthreads();
    if (tid == 0 && mine == 0) engine_stamp(e, k, kStampDesc);
    const uint32_t tpc = d.a.tiles_per_chunk;
    const uint32_t total = tpc * d.a.n_chunks;
    const uint32_t kind = d.kind;
    // a share is `share` neighbouring tiles: one copy of that many times the length when they lie in one chunk
    const uint32_t share = d.share;
    const bool whole = tpc % share == 0;
    if (kind != kEngineRecv) {
      // user buffers -> staging windows and, from the same registers, on: into the receive buffers (kEngineLoop, the
      // descriptor's onward buffers) or into the same lane and offset of the receiving process's landing windows
      // (kEngineSend).  One pass, nothing read back.
      for (uint32_t sh = mine; sh * share < total; sh += W) {
        const uint32_t t0 = sh * share;
        if (whole) fused_tile<3, 12>(d.a, t0 % tpc, t0 / tpc, share);
        else for (uint32_t t = t0; t < total && t < t0 + share; ++t) fused_tile<3, 12>(d.a, t % tpc, t / tpc);
      }
    } else {
      // landing windows -> receive buffers.  Another process's kernel wrote the windows (written through, or written
      // back at the end of its kernel): loaded at system scope, whatever this XCD's L2 has kept of the set's last use.
      for (uint32_t sh = mine; sh * share < total; sh += W) {
        const uint32_t t0 = sh * share;
        if (whole) fused_tile<1, 12>(d.a, t0 % tpc, t0 / tpc, share);
        else for (uint32_t t = t0; t < total && t < t0 + share; ++t) fused_tile<1, 12>(d.a, t % tpc, t / tpc);
      }
    }
    // Every thread waits until its stores have been written through and its loads have returned: the wave's memory
    // counter at zero.  (Written out: no fence stands for exactly this.  A release at workgroup scope waits for nothing,
    // a workgroup's accesses being ordered by the L1 they share; one at agent scope adds the L2 write-back that mode 4
    // is there to avoid.)  Behind the barrier the whole share is in memory, and the count says so.  The last worker to leave has read a count that every other one incremented after the same wait,
    // so the batch is in memory when it tells the host.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0) {
      if (mine == 0) engine_stamp(e, k, kStampMoved);
      const uint64_t before = __hip_atomic_fetch_add(cnt, (uint64_t)1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if ((((uint32_t)before + 1) & kEngineCountMask) == own_target) {
        __hip_atomic_store(&e.hctl->done[k % kEngineDevRing], k + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        // once the word is out (the store acknowledged), the slot may go to batch k + ring: the word of a slot is
        // never stored out of order
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __hip_atomic_store(&e.dctl->freed[k % kEngineDevRing], k + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        engine_stamp(e, k, kStampDone);
      }
    }
  }
}

}  // namespace

// One launch per (direction, streaming mode) pair that the policy can ask for: striping / gathering with modes
// 0, 1, 3, reassembly / scattering with 0, 2, 3 (fl_stream_mode returns no other).  EXTRA carries trailing
// template arguments.
#define FL_LAUNCH_COPY(NAME, EXTRA, dir, mode, grid, s, a)                                  \
  do {                                                                                      \
    if ((dir) == 0) {                                                                       \
      if ((mode) == 0) FL_LAUNCH((NAME<0, 0 EXTRA>), grid, dim3(kCopyBlock), 0, s, a);      \
      else if ((mode) == 1) FL_LAUNCH((NAME<0, 1 EXTRA>), grid, dim3(kCopyBlock), 0, s, a); \
      else FL_LAUNCH((NAME<0, 3 EXTRA>), grid, dim3(kCopyBlock), 0, s, a);                  \
    } else {                                                                                \
      if ((mode) == 0) FL_LAUNCH((NAME<1, 0 EXTRA>), grid, dim3(kCopyBlock), 0, s, a);      \
      else if ((mode) == 2) FL_LAUNCH((NAME<1, 2 EXTRA>), grid, dim3(kCopyBlock), 0, s, a); \
      else FL_LAUNCH((NAME<1, 3 EXTRA>), grid, dim3(kCopyBlock), 0, s, a);                  \
    }                                                                                       \
  } while (0)
#define FL_NO_EXTRA

extern "C" {

static int check_windows(const flh_windows* win) {
  if (!win) return fl_set_error(FLH_E_ARG, "null windows");
  if (win->n_lanes == 0 || win->n_lanes > FLH_MAX_LANES) return fl_set_error(FLH_E_ARG, "windows.n_lanes %u not in 1..%d", win->n_lanes, FLH_MAX_LANES);
  for (uint32_t l = 0; l < win->n_lanes; ++l)
    if (!win->base[l] && win->cap[l]) return fl_set_error(FLH_E_ARG, "window %u has capacity but no base", l);
  return FLH_OK;
}

static int launch_copy(int dir, void* user, uint64_t user_bytes, const flh_windows* win, const flh_chunk_desc* d_table,
                       const flh_sched_hdr* d_hdr, const flh_sched_hdr* h_hdr, uint32_t n_chunks_max, uint32_t tile_bytes, int32_t* d_status, void* stream) {
  int rc = check_windows(win);
  if (rc) return rc;
  if (!d_hdr || !d_status) return fl_set_error(FLH_E_ARG, "d_hdr and d_status are required");
  if (n_chunks_max && !d_table) return fl_set_error(FLH_E_ARG, "d_table missing");
  if (tile_bytes == 0 || tile_bytes % 128) return fl_set_error(FLH_E_ARG, "tile_bytes %u must be a positive multiple of 128", tile_bytes);
  if (user_bytes && !user) return fl_set_error(FLH_E_ARG, "user buffer missing");
  if (n_chunks_max == 0) return FLH_OK;
  rc = fl_need_init();
  if (rc) return rc;
  fl_prof().kid = dir == 0 ? 2 : 3;
  CopyArgs a;
  a.user = (uint8_t*)user;
  a.user_bytes = user_bytes;
  a.win = *win;
  a.table = d_table;
  a.hdr = d_hdr;
  a.status = d_status;
  a.n_chunks_max = n_chunks_max;
  a.tile_bytes = tile_bytes;
  a.has_hint = h_hdr != nullptr;
  a.hint_total_tiles = h_hdr ? h_hdr->total_tiles : 0;
  a.hint_n_chunks = h_hdr ? h_hdr->n_chunks : 0;
  a.hint_uniform_tiles = h_hdr ? h_hdr->uniform_tiles : 0;
  a.xcd = 0;
  const uint64_t max_tiles = h_hdr ? h_hdr->total_tiles : user_bytes / tile_bytes + n_chunks_max;
  if (max_tiles == 0) return FLH_OK;
  hipStream_t s = (hipStream_t)stream;
  const int mode = fl_stream_mode(dir, user_bytes);
  if (h_hdr && h_hdr->uniform_tiles && h_hdr->n_chunks <= 65535 && h_hdr->n_chunks <= n_chunks_max && g_copy_uniform_grid) {
    const dim3 grid(h_hdr->uniform_tiles, h_hdr->n_chunks);
    a.xcd = fl_xcd_map(grid.x, grid.y);
    FL_LAUNCH_COPY(fl_copy_uniform, FL_NO_EXTRA, dir, mode, grid, s, a);
    FL_HIP(hipGetLastError());
    return FLH_OK;
  }
  const dim3 grid(fl_copy_grid(max_tiles));
  a.xcd = grid.x == max_tiles ? fl_xcd_full(grid.x) : 0;   // only with one workgroup per tile
  FL_LAUNCH_COPY(fl_copy_tiles, FL_NO_EXTRA, dir, mode, grid, s, a);
  FL_HIP(hipGetLastError());
  return FLH_OK;
}

static int launch_desc(int dir, void* user, uint64_t user_bytes, const flh_windows* win, const flh_tile_desc* d_tiles, uint32_t tiles_cap,
                       const flh_sched_hdr* d_hdr, const flh_sched_hdr* h_hdr, int32_t* d_status, void* stream) {
  int rc = check_windows(win);
  if (rc) return rc;
  if (!d_tiles || tiles_cap == 0) return fl_set_error(FLH_E_ARG, "tile descriptors missing");
  if (!d_status || (!d_hdr && !h_hdr)) return fl_set_error(FLH_E_ARG, "d_status and a header (device or host copy) are required");
  if (user_bytes && !user) return fl_set_error(FLH_E_ARG, "user buffer missing");
  if (h_hdr && h_hdr->total_tiles > tiles_cap) return fl_set_error(FLH_E_RANGE, "the table has %u tiles, the descriptor array holds %u", h_hdr->total_tiles, tiles_cap);
  const uint32_t grid = h_hdr ? h_hdr->total_tiles : tiles_cap;
  if (grid == 0) return FLH_OK;
  rc = fl_need_init();
  if (rc) return rc;
  fl_prof().kid = dir == 0 ? 2 : 3;
  DescArgs a;
  a.user = (uint8_t*)user;
  a.user_bytes = user_bytes;
  a.win = *win;
  a.tiles = d_tiles;
  a.hdr = d_hdr;
  a.status = d_status;
  a.tiles_cap = tiles_cap;
  a.has_hint = h_hdr != nullptr;
  a.hint_total_tiles = h_hdr ? h_hdr->total_tiles : 0;
  a.xcd = fl_xcd_full(grid);
  hipStream_t s = (hipStream_t)stream;
  const int mode = fl_stream_mode(dir, user_bytes);
  FL_LAUNCH_COPY(fl_copy_desc, FL_NO_EXTRA, dir, mode, dim3(grid), s, a);
  FL_HIP(hipGetLastError());
  return FLH_OK;
}

int flh_stripe_tiles(const void* d_src, uint64_t src_bytes, const flh_windows* win, const flh_tile_desc* d_tiles,
                     uint32_t tiles_cap, const flh_sched_hdr* d_hdr, const flh_sched_hdr* h_hdr, int32_t* d_status, void* stream) {
  return launch_desc(0, (void*)d_src, src_bytes, win, d_tiles, tiles_cap, d_hdr, h_hdr, d_status, stream);
}

int flh_reassemble_tiles(void* d_dst, uint64_t dst_bytes, const flh_windows* win, const flh_tile_desc* d_tiles,
                         uint32_t tiles_cap, const flh_sched_hdr* d_hdr, const flh_sched_hdr* h_hdr, int32_t* d_status, void* stream) {
  return launch_desc(1, d_dst, dst_bytes, win, d_tiles, tiles_cap, d_hdr, h_hdr, d_status, stream);
}

int flh_stripe(const void* d_src, uint64_t src_bytes, const flh_windows* win, const flh_chunk_desc* d_table,
               const flh_sched_hdr* d_hdr, const flh_sched_hdr* h_hdr, uint32_t n_chunks_max, uint32_t tile_bytes,
               int32_t* d_status, void* stream) {
  return launch_copy(0, (void*)d_src, src_bytes, win, d_table, d_hdr, h_hdr, n_chunks_max, tile_bytes, d_status, stream);
}

int flh_reassemble(void* d_dst, uint64_t dst_bytes, const flh_windows* win, const flh_chunk_desc* d_table,
                   const flh_sched_hdr* d_hdr, const flh_sched_hdr* h_hdr, uint32_t n_chunks_max, uint32_t tile_bytes,
                   int32_t* d_status, void* stream) {
  return launch_copy(1, d_dst, dst_bytes, win, d_table, d_hdr, h_hdr, n_chunks_max, tile_bytes, d_status, stream);
}

// argument checks and everything of FusedArgs that follows from the parameters; returns 1 when there is nothing to do
static int fill_fused(FusedArgs& a, int dir, const flh_windows* win, const flh_uniform_params* u, flh_chunk_desc* d_table,
                      flh_sched_hdr* d_hdr, int32_t* d_status, const flh_windows* carry = nullptr, bool onward = false) {
  int rc = check_windows(win);
  if (rc) return rc;
  if (carry) {   // (the caller's argument block holds the windows themselves)
    if (dir != 0) return fl_set_error(FLH_E_ARG, "only the striping side carries its tiles on");
    rc = check_windows(carry);
    if (rc) return rc;
    if (carry->n_lanes != win->n_lanes) return fl_set_error(FLH_E_ARG, "%u landing windows for %u staging windows", carry->n_lanes, win->n_lanes);
  }
  if (!u || !d_status) return fl_set_error(FLH_E_ARG, "parameters and d_status are required");
  if (u->n_lanes == 0 || u->n_lanes > FLH_MAX_LANES || u->n_lanes != win->n_lanes) return fl_set_error(FLH_E_ARG, "n_lanes %u does not match the windows' %u", u->n_lanes, win->n_lanes);
  if (u->chunk_bytes == 0) return fl_set_error(FLH_E_ARG, "chunk_bytes must be > 0");
  if (u->tile_bytes == 0 || u->tile_bytes % 128) return fl_set_error(FLH_E_ARG, "tile_bytes %u must be a positive multiple of 128", u->tile_bytes);
  if (u->total_bytes == 0) return 1;
  const uint64_t n = (u->total_bytes + u->chunk_bytes - 1) / u->chunk_bytes;
  if (n > 65535) return fl_set_error(FLH_E_ARG, "%llu chunks exceed the 65535 one launch can name; split the message", (unsigned long long)n);
  rc = fl_need_init();
  if (rc) return rc;
  if (onward && (dir != 0 || carry)) return fl_set_error(FLH_E_ARG, "a launch delivers into receive buffers or carries into landing windows, from the striping side");
  fl_prof().kid = dir == 0 ? (onward ? 7 : 2) : 3;
  const bool last = dir == 1 || carry || onward;   // the launch that ends the path on this side reports
  a.user = nullptr;
  a.user_bytes = 0;
  a.win = *win;
  a.table = dir == 0 ? d_table : nullptr;
  a.hdr = dir == 0 ? d_hdr : nullptr;
  a.status = d_status;
  a.done_word = last ? u->d_done_word : nullptr;
  a.done_count = last ? u->d_done_count : nullptr;
  a.done_value = u->done_value;
  if (a.done_word && !a.done_count) return fl_set_error(FLH_E_ARG, "d_done_word needs d_done_count");
  a.start_word = u->d_start_word;
  a.start_value = u->start_value;
  a.pad_start = 0;
  a.total_bytes = u->total_bytes;
  a.src_base = u->src_base;
  a.quanta_before = u->epoch_bytes / u->chunk_bytes;
  a.chunk_bytes = u->chunk_bytes;
  a.n_chunks = (uint32_t)n;
  a.n_lanes = u->n_lanes;
  a.tile_bytes = u->tile_bytes;
  a.tiles_per_chunk = (u->chunk_bytes + u->tile_bytes - 1) / u->tile_bytes;
  a.xcd_map = fl_xcd_map(a.tiles_per_chunk, (uint32_t)n);
  // once the message no longer fits the Infinity Cache, write every window front to back
  a.dest_order = dir == 0 && (g_dest_order < 0 ? u->total_bytes > kWindowsCacheableBytes : g_dest_order != 0);
  for (int l = 0; l < FLH_MAX_LANES; ++l) a.credits[l] = (uint32_t)l < u->n_lanes ? u->credits[l] : 0;
  {
    // the row as the kernel sees it (equal credits stand in for an all-zero row), then the host-side constants
    uint64_t pfx[FLH_MAX_LANES], W = 0;
    for (uint32_t l = 0; l < u->n_lanes; ++l) { W += u->credits[l]; pfx[l] = W; }
    if (W == 0) { for (uint32_t l = 0; l < u->n_lanes; ++l) pfx[l] = l + 1; W = u->n_lanes; }
    a.fast = W <= 0xffffffffull && a.quanta_before + n <= 0xffffffffull && g_fused_fast;
    a.magic = a.fast && W >= 2 ? ~0ull / W + 1 : 0;   // ceil(2^64 / W); W = 1 (one lane named outright) needs no division
    for (int l = 0; l < FLH_MAX_LANES; ++l) a.cnt0[l] = 0;
    for (int l = 0; l <= FLH_MAX_LANES; ++l) a.pfx_ex[l] = l == 0 ? 0 : (uint32_t)((uint32_t)l <= u->n_lanes ? pfx[l - 1] : W);
    if (a.fast) {
      const uint64_t full = a.quanta_before / W, rem = a.quanta_before % W;
      for (uint32_t l = 0; l < u->n_lanes; ++l) {
        const uint64_t K = l ? pfx[l - 1] : 0, cl = pfx[l] - K;
        const uint64_t part = rem <= K ? 0 : (rem - K < cl ? rem - K : cl);
        a.cnt0[l] = (uint32_t)(full * cl + part);
      }
    }
  }
  return FLH_OK;
}

extern "C++" {
template <class Args>
static int launch_fused_args(int dir, const Args& a, int mode, void* stream, void* done_event) {
  const dim3 grid(a.tiles_per_chunk, a.n_chunks);
  hipStream_t s = (hipStream_t)stream;
  hipEvent_t ev = dir == 1 || has_carry<Args>::value ? (hipEvent_t)done_event : nullptr;
#define FL_ARGS_EXTRA , Args
  if (dir == 0) {
    if (mode == 0) FL_LAUNCH_EV((fl_copy_uniform_fused<0, 0 FL_ARGS_EXTRA>), grid, dim3(kCopyBlock), 0, s, ev, a);
    else if (mode == 1) FL_LAUNCH_EV((fl_copy_uniform_fused<0, 1 FL_ARGS_EXTRA>), grid, dim3(kCopyBlock), 0, s, ev, a);
    else if (mode == 3) FL_LAUNCH_EV((fl_copy_uniform_fused<0, 3 FL_ARGS_EXTRA>), grid, dim3(kCopyBlock), 0, s, ev, a);
    else if constexpr (has_carry<Args>::value) {
      // a launch with two destinations: bit 1 for the stores that go on, bit 4 for the stores into the staging windows
      if (mode == 2) FL_LAUNCH_EV((fl_copy_uniform_fused<0, 2 FL_ARGS_EXTRA>), grid, dim3(kCopyBlock), 0, s, ev, a);
      else if (mode == 16) FL_LAUNCH_EV((fl_copy_uniform_fused<0, 16 FL_ARGS_EXTRA>), grid, dim3(kCopyBlock), 0, s, ev, a);
      else if (mode == 18) FL_LAUNCH_EV((fl_copy_uniform_fused<0, 18 FL_ARGS_EXTRA>), grid, dim3(kCopyBlock), 0, s, ev, a);
      else if (mode == 19) FL_LAUNCH_EV((fl_copy_uniform_fused<0, 19 FL_ARGS_EXTRA>), grid, dim3(kCopyBlock), 0, s, ev, a);
      else return fl_set_error(FLH_E_ARG, "streaming mode %d of a launch with two destinations is not built", mode);
    }
    else return fl_set_error(FLH_E_ARG, "streaming mode %d of a striping launch is not built", mode);
  } else if constexpr (!has_carry<Args>::value) {   // (only the striping side carries)
    if (mode == 0) FL_LAUNCH_EV((fl_copy_uniform_fused<1, 0 FL_ARGS_EXTRA>), grid, dim3(kCopyBlock), 0, s, ev, a);
    else if (mode == 2) FL_LAUNCH_EV((fl_copy_uniform_fused<1, 2 FL_ARGS_EXTRA>), grid, dim3(kCopyBlock), 0, s, ev, a);
    else FL_LAUNCH_EV((fl_copy_uniform_fused<1, 3 FL_ARGS_EXTRA>), grid, dim3(kCopyBlock), 0, s, ev, a);
  }
#undef FL_ARGS_EXTRA
  FL_HIP(hipGetLastError());
  return FLH_OK;
}
}  // extern "C++"

// Streaming mode of a launch that stages and delivers: the windows are written and not read again and the receive
// buffer is read by whoever comes next, so the stores stream from the size on from which the reassembly's do, the loads
// from the size on from which the striping's do.
static int deliver_mode(uint64_t total_bytes) {
  if (g_stream_force_deliver >= 0) return g_stream_force_deliver;
  // (the windows stay cacheable for as long as the striping launch's do: rewritten by the next message before the
  // Infinity Cache has given them up, they cost no traffic to memory at all)
  const int out = fl_stream_mode(0, total_bytes);
  return (out & 1) | (fl_stream_mode(1, total_bytes) & 2) | ((out & 2) ? 16 : 0);
}
// ... that carries into landing windows, which the receiving process reads next: both kinds of window alike
static int carry_mode(uint64_t total_bytes) {
  const int out = fl_stream_mode(0, total_bytes);
  return out | ((out & 2) ? 16 : 0);
}

static int launch_fused(int dir, void* user, uint64_t user_bytes, const flh_windows* win, const flh_uniform_params* u,
                        flh_chunk_desc* d_table, flh_sched_hdr* d_hdr, int32_t* d_status, void* stream, const flh_windows* carry = nullptr,
                        void* onward = nullptr, uint64_t onward_bytes = 0) {
  FusedCarryArgs a;
  const int rc = fill_fused(a, dir, win, u, d_table, d_hdr, d_status, carry, onward != nullptr);
  if (rc) return rc < 0 ? rc : FLH_OK;
  if (!user) return fl_set_error(FLH_E_ARG, "user buffer missing");
  a.user = (uint8_t*)user;
  a.user_bytes = user_bytes;
  if (!carry && !onward) return launch_fused_args(dir, static_cast<const FusedArgs&>(a), fl_stream_mode(dir, u->total_bytes), stream, u->done_event);
  memset(&a.carry, 0, sizeof(a.carry));
  if (carry) a.carry = *carry;
  a.onward = (uint8_t*)onward;
  a.onward_bytes = onward_bytes;
  return launch_fused_args(dir, a, onward ? deliver_mode(u->total_bytes) : carry_mode(u->total_bytes), stream, u->done_event);
}

// What a batch comes to: its segments as the kernel takes them, and where each lane's window ends up.
struct BatchPlan {
  uint32_t n_seg;
  uint32_t n_chunks;
  uint32_t first[FLH_BATCH_MAX];
  uint8_t seg_of[FLH_BATCH_MAX];
  BatchSeg seg[FLH_SEG_MAX];
  uint64_t seg_base[FLH_SEG_MAX][FLH_MAX_LANES];
  uint64_t lane_end[FLH_MAX_LANES];
};

static int plan_batch(const flh_batch_params* b, BatchPlan& pl) {
  if (!b) return fl_set_error(FLH_E_ARG, "null batch");
  if (b->n_req == 0 || b->n_req > FLH_BATCH_MAX) return fl_set_error(FLH_E_ARG, "n_req %u not in 1..%d", b->n_req, FLH_BATCH_MAX);
  if (b->n_seg > FLH_SEG_MAX) return fl_set_error(FLH_E_ARG, "n_seg %u not in 0..%d", b->n_seg, FLH_SEG_MAX);
  const flh_uniform_params& u = b->u;
  if (u.n_lanes == 0 || u.n_lanes > FLH_MAX_LANES) return fl_set_error(FLH_E_ARG, "n_lanes %u not in 1..%d", u.n_lanes, FLH_MAX_LANES);
  if (u.chunk_bytes == 0) return fl_set_error(FLH_E_ARG, "chunk_bytes must be > 0");
  memset(&pl, 0, sizeof(pl));
  pl.n_seg = b->n_seg ? b->n_seg : 1;
  uint32_t q = 0, chunk_at = 0;
  uint64_t sum = 0;
  for (uint32_t k = 0; k < pl.n_seg; ++k) {
    const uint32_t nq = b->n_seg ? b->seg[k].n_req : b->n_req;
    const uint32_t* credits = b->n_seg ? b->seg[k].credits : u.credits;
    const uint64_t epoch_bytes = b->n_seg ? b->seg[k].epoch_bytes : u.epoch_bytes;
    if (nq == 0 || q + nq > b->n_req) return fl_set_error(FLH_E_ARG, "segment %u holds %u requests, %u are left", k, nq, b->n_req - q);
    BatchSeg& g = pl.seg[k];
    uint64_t seg_bytes = 0;
    for (uint32_t i = 0; i < nq; ++i, ++q) {
      if (b->bytes[q] == 0) return fl_set_error(FLH_E_ARG, "request %u of the batch has no bytes", q);
      if (i + 1 < nq && b->bytes[q] % u.chunk_bytes) return fl_set_error(FLH_E_ARG, "request %u of the batch is not a whole number of chunks", q);
      pl.first[q] = chunk_at + (uint32_t)(seg_bytes / u.chunk_bytes);
      pl.seg_of[q] = (uint8_t)k;
      seg_bytes += b->bytes[q];
    }
    const uint64_t n = (seg_bytes + u.chunk_bytes - 1) / u.chunk_bytes;
    FlCreditRow row;
    fl_row_make(credits, u.n_lanes, row);
    const uint64_t x0 = epoch_bytes / u.chunk_bytes;
    if (row.W > 0xffffffffull || x0 + n > 0xffffffffull || chunk_at + n > 65535)
      return fl_set_error(FLH_E_ARG, "segment %u: a credit row that sums past 2^32 - 1, a credit epoch of 2^32 quanta or more, or more than 65535 chunks in the launch", k);
    g.magic = row.W >= 2 ? ~0ull / row.W + 1 : 0;
    g.quanta_before = (uint32_t)x0;
    g.first_chunk = chunk_at;
    g.n_chunks = (uint32_t)n;
    g.short_by = (uint32_t)(n * u.chunk_bytes - seg_bytes);
    g.zero = row.zero;
    for (uint32_t l = 0; l <= FLH_MAX_LANES; ++l) g.pfx_ex[l] = (uint32_t)row.K[l];
    uint64_t lane_bytes[FLH_MAX_LANES];
    uint32_t lane_chunks[FLH_MAX_LANES];
    fl_row_lane_totals(row, x0, seg_bytes, u.chunk_bytes, lane_bytes, lane_chunks);
    for (uint32_t l = 0; l < FLH_MAX_LANES; ++l) {
      g.cnt0[l] = l < u.n_lanes ? (uint32_t)fl_row_before(row, l, x0) : 0;
      const uint64_t base = (pl.lane_end[l] + 127) / 128 * 128;   // the alignment of the reference's per-QP pieces (plugin.cc:1467)
      if (base / 128 > 0xffffffffull) return fl_set_error(FLH_E_ARG, "segment %u starts beyond 512 GiB in a window", k);
      g.base128[l] = (uint32_t)(base / 128);
      pl.seg_base[k][l] = base;
      if (lane_chunks[l]) pl.lane_end[l] = base + lane_bytes[l];
    }
    chunk_at += (uint32_t)n;
    sum += seg_bytes;
  }
  if (q != b->n_req) return fl_set_error(FLH_E_ARG, "the segments hold %u requests, the batch %u", q, b->n_req);
  if (sum != u.total_bytes) return fl_set_error(FLH_E_ARG, "the requests hold %llu bytes, the parameters say %llu", (unsigned long long)sum, (unsigned long long)u.total_bytes);
  for (uint32_t r = b->n_req; r < FLH_BATCH_MAX; ++r) pl.first[r] = 0xffffffffu;
  pl.n_chunks = chunk_at;
  return FLH_OK;
}

int flh_batch_layout(const flh_batch_params* b, uint64_t* lane_end, uint64_t* seg_base) {
  BatchPlan pl;
  const int rc = plan_batch(b, pl);
  if (rc) return rc;
  if (lane_end) memcpy(lane_end, pl.lane_end, sizeof(pl.lane_end));
  if (seg_base) memcpy(seg_base, pl.seg_base, sizeof(pl.seg_base));
  return FLH_OK;
}

static int launch_batch(int dir, const flh_batch_params* b, const flh_windows* win, flh_chunk_desc* d_table, flh_sched_hdr* d_hdr,
                        int32_t* d_status, void* stream, const flh_windows* carry = nullptr, bool onward = false) {
  BatchPlan pl;
  int rc = plan_batch(b, pl);
  if (rc) return rc;
  FusedBatchCarryArgs a;
  // fill_fused sees the launch as one message of n_chunks whole chunks (grid, tiles per chunk, checks); the credit row
  // it prepares goes unused, every segment brings its own
  flh_uniform_params u = b->u;
  u.total_bytes = (uint64_t)pl.n_chunks * b->u.chunk_bytes;
  u.epoch_bytes = 0;
  rc = fill_fused(a, dir, win, &u, d_table, d_hdr, d_status, carry, onward);
  if (rc) return rc < 0 ? rc : FLH_OK;
  a.total_bytes = b->u.total_bytes;
  a.dest_order = 0;
  a.src_base = 0;
  a.n_req = b->n_req;
  a.n_seg = pl.n_seg;
  for (uint32_t q = 0; q < FLH_BATCH_MAX; ++q) {
    a.first[q] = pl.first[q];
    a.seg_of[q] = pl.seg_of[q];
    a.req_user[q] = nullptr;
    a.req_bytes[q] = 0;
    a.onward[q] = nullptr;
    if (q >= b->n_req) continue;
    void* p = dir == 0 ? (void*)b->d_src[q] : b->d_dst[q];
    if (!p || (onward && !b->d_dst[q])) return fl_set_error(FLH_E_ARG, "request %u of the batch has no buffer", q);
    a.req_user[q] = (uint8_t*)p;
    a.req_bytes[q] = b->bytes[q];
    if (onward) a.onward[q] = (uint8_t*)b->d_dst[q];
  }
  for (uint32_t k = 0; k < FLH_SEG_MAX; ++k) a.seg[k] = pl.seg[k];
  if (!carry && !onward) return launch_fused_args(dir, static_cast<const FusedBatchArgs&>(a), fl_stream_mode(dir, b->u.total_bytes), stream, b->u.done_event);
  memset(&a.carry, 0, sizeof(a.carry));
  if (carry) a.carry = *carry;
  return launch_fused_args(dir, a, onward ? deliver_mode(b->u.total_bytes) : carry_mode(b->u.total_bytes), stream, b->u.done_event);
}

static int launch_fused_pages(int dir, void* pool, uint64_t pool_pages, const uint32_t* d_page_table, uint32_t page_bytes,
                              const flh_windows* win, const flh_uniform_params* u, flh_chunk_desc* d_table, flh_sched_hdr* d_hdr,
                              int32_t* d_status, void* stream) {
  FusedPageArgs a;
  const int rc = fill_fused(a, dir, win, u, d_table, d_hdr, d_status);
  if (rc) return rc < 0 ? rc : FLH_OK;
  if (!pool || !d_page_table) return fl_set_error(FLH_E_ARG, "pool and page table are required");
  if (page_bytes == 0 || page_bytes % u->tile_bytes) return fl_set_error(FLH_E_ARG, "tile_bytes %u must divide page_bytes %u", u->tile_bytes, page_bytes);
  if (u->chunk_bytes % page_bytes || u->src_base % page_bytes) return fl_set_error(FLH_E_ARG, "chunk_bytes and src_base must be multiples of page_bytes %u", page_bytes);
  fl_prof().kid = dir == 0 ? 4 : 5;
  a.user = (uint8_t*)pool;
  a.user_bytes = pool_pages * (uint64_t)page_bytes;
  a.page_table = d_page_table;
  a.pool_pages = pool_pages;
  a.n_pages = (u->src_base + u->total_bytes + page_bytes - 1) / page_bytes;
  a.page_bytes = page_bytes;
  a.page_shift = (page_bytes & (page_bytes - 1)) == 0 ? __builtin_ctz(page_bytes) : -1;
  return launch_fused_args(dir, a, fl_stream_mode(dir, u->total_bytes), stream, u->done_event);
}

int flh_gather_pages_uniform(const void* d_pool, uint64_t pool_pages, const uint32_t* d_page_table, uint32_t page_bytes,
                             const flh_windows* win, const flh_uniform_params* u, flh_chunk_desc* d_table_out,
                             flh_sched_hdr* d_hdr_out, int32_t* d_status, void* stream) {
  return launch_fused_pages(0, (void*)d_pool, pool_pages, d_page_table, page_bytes, win, u, d_table_out, d_hdr_out, d_status, stream);
}

int flh_scatter_pages_uniform(void* d_pool, uint64_t pool_pages, const uint32_t* d_page_table, uint32_t page_bytes,
                              const flh_windows* win, const flh_uniform_params* u, int32_t* d_status, void* stream) {
  return launch_fused_pages(1, d_pool, pool_pages, d_page_table, page_bytes, win, u, nullptr, nullptr, d_status, stream);
}

int flh_stripe_batch(const flh_batch_params* b, const flh_windows* win, flh_chunk_desc* d_table_out, flh_sched_hdr* d_hdr_out,
                     int32_t* d_status, void* stream) {
  return launch_batch(0, b, win, d_table_out, d_hdr_out, d_status, stream);
}

int flh_reassemble_batch(const flh_batch_params* b, const flh_windows* win, int32_t* d_status, void* stream) {
  return launch_batch(1, b, win, nullptr, nullptr, d_status, stream);
}

int flh_stripe_uniform(const void* d_src, uint64_t src_bytes, const flh_windows* win, const flh_uniform_params* u,
                       flh_chunk_desc* d_table_out, flh_sched_hdr* d_hdr_out, int32_t* d_status, void* stream) {
  return launch_fused(0, (void*)d_src, src_bytes, win, u, d_table_out, d_hdr_out, d_status, stream);
}

int flh_stage_deliver_uniform(const void* d_src, uint64_t src_bytes, void* d_dst, uint64_t dst_bytes, const flh_windows* win,
                              const flh_uniform_params* u, flh_chunk_desc* d_table_out, flh_sched_hdr* d_hdr_out, int32_t* d_status, void* stream) {
  if (!d_dst) return fl_set_error(FLH_E_ARG, "receive buffer missing");
  return launch_fused(0, (void*)d_src, src_bytes, win, u, d_table_out, d_hdr_out, d_status, stream, nullptr, d_dst, dst_bytes);
}

int flh_stripe_uniform_carry(const void* d_src, uint64_t src_bytes, const flh_windows* win, const flh_windows* landing,
                             const flh_uniform_params* u, flh_chunk_desc* d_table_out, flh_sched_hdr* d_hdr_out, int32_t* d_status, void* stream) {
  if (!landing) return fl_set_error(FLH_E_ARG, "null landing windows");
  return launch_fused(0, (void*)d_src, src_bytes, win, u, d_table_out, d_hdr_out, d_status, stream, landing);
}

int flh_stage_deliver_batch(const flh_batch_params* b, const flh_windows* win, flh_chunk_desc* d_table_out, flh_sched_hdr* d_hdr_out,
                            int32_t* d_status, void* stream) {
  return launch_batch(0, b, win, d_table_out, d_hdr_out, d_status, stream, nullptr, true);
}

int flh_stripe_batch_carry(const flh_batch_params* b, const flh_windows* win, const flh_windows* landing, flh_chunk_desc* d_table_out,
                           flh_sched_hdr* d_hdr_out, int32_t* d_status, void* stream) {
  if (!landing) return fl_set_error(FLH_E_ARG, "null landing windows");
  return launch_batch(0, b, win, d_table_out, d_hdr_out, d_status, stream, landing);
}

int flh_reassemble_uniform(void* d_dst, uint64_t dst_bytes, const flh_windows* win, const flh_uniform_params* u,
                           int32_t* d_status, void* stream) {
  return launch_fused(1, d_dst, dst_bytes, win, u, nullptr, nullptr, d_status, stream);
}

static int launch_pages(int dir, void* pool, uint64_t pool_pages, const uint32_t* d_page_table, uint32_t page_bytes,
                        uint32_t pages_per_chunk, const flh_windows* win, const flh_chunk_desc* d_table, uint32_t n_chunks,
                        int use_lds, int32_t* d_status, void* stream) {
  int rc = check_windows(win);
  if (rc) return rc;
  if (!pool || !d_page_table || !d_status) return fl_set_error(FLH_E_ARG, "pool, page table and status are required");
  if (page_bytes == 0 || pages_per_chunk == 0) return fl_set_error(FLH_E_ARG, "page_bytes and pages_per_chunk must be > 0");
  if (n_chunks == 0) return FLH_OK;
  if (!d_table) return fl_set_error(FLH_E_ARG, "d_table missing");
  rc = fl_need_init();
  if (rc) return rc;
  fl_prof().kid = dir == 0 ? 4 : 5;
  PageArgs a;
  a.pool = (uint8_t*)pool;
  a.pool_pages = pool_pages;
  a.page_table = d_page_table;
  a.win = *win;
  a.table = d_table;
  a.status = d_status;
  a.n_chunks = n_chunks;
  a.page_bytes = page_bytes;
  a.pages_per_chunk = pages_per_chunk;
  const uint32_t sub = use_lds ? kLdsStage : FLH_TILE_BYTES;
  a.sub_bytes = page_bytes < sub ? page_bytes : sub;
  a.subs_per_page = (page_bytes + a.sub_bytes - 1) / a.sub_bytes;
  a.page_shift = (page_bytes & (page_bytes - 1)) == 0 ? __builtin_ctz(page_bytes) : -1;
  const uint64_t per_chunk = (uint64_t)pages_per_chunk * a.subs_per_page;
  if (per_chunk > 0x7fffffffull) return fl_set_error(FLH_E_ARG, "pages_per_chunk %u is too large for one launch", pages_per_chunk);
  hipStream_t s = (hipStream_t)stream;
  const int mode = fl_stream_mode(dir, (uint64_t)n_chunks * pages_per_chunk * page_bytes);
  const dim3 grid3((uint32_t)per_chunk, n_chunks < 65535 ? n_chunks : 65535);
  a.xcd_map = grid3.y == n_chunks ? fl_xcd_map(grid3.x, grid3.y) : 0;   // only with one grid row per chunk
#define FL_LDS_ON , true
#define FL_LDS_OFF , false
  if (use_lds) FL_LAUNCH_COPY(fl_page_tiles, FL_LDS_ON, dir, mode, grid3, s, a);
  else FL_LAUNCH_COPY(fl_page_tiles, FL_LDS_OFF, dir, mode, grid3, s, a);
#undef FL_LDS_ON
#undef FL_LDS_OFF
  FL_HIP(hipGetLastError());
  return FLH_OK;
}

int flh_gather_pages(const void* d_pool, uint64_t pool_pages, const uint32_t* d_page_table, uint32_t page_bytes,
                     uint32_t pages_per_chunk, const flh_windows* win, const flh_chunk_desc* d_table, uint32_t n_chunks,
                     int use_lds, int32_t* d_status, void* stream) {
  return launch_pages(0, (void*)d_pool, pool_pages, d_page_table, page_bytes, pages_per_chunk, win, d_table, n_chunks, use_lds, d_status, stream);
}

int flh_scatter_pages(void* d_pool, uint64_t pool_pages, const uint32_t* d_page_table, uint32_t page_bytes,
                      uint32_t pages_per_chunk, const flh_windows* win, const flh_chunk_desc* d_table, uint32_t n_chunks,
                      int use_lds, int32_t* d_status, void* stream) {
  return launch_pages(1, d_pool, pool_pages, d_page_table, page_bytes, pages_per_chunk, win, d_table, n_chunks, use_lds, d_status, stream);
}

// ---- lane engine, host side ---------------------------------------------------------------------------------
struct flh_engine {
  int device;
  uint32_t workers;
  uint32_t host_slots;
  uint32_t sets;
  hipStream_t stream;
  uint8_t* h_ring;          // pinned, mapped
  uint8_t* d_ring_host;     // the same ring as the device addresses it
  EngineHostCtl* h_ctl;
  EngineHostCtl* d_ctl_host;
  uint8_t* dev_ring;
  EngineDevCtl* dctl;
  uint64_t submitted;       // batches written into the ring
  uint64_t completed;       // batches known complete, in order (atomic; moved forward by whoever looks)
  uint64_t launches;        // engine kernels started
  uint64_t idle_us, wait_us, resident_us;
  uint64_t* d_trace;        // null unless the engine was created with flh_tune("engine_trace") set
  uint32_t trace_slots;
};

int flh_engine_create(int device, uint32_t workgroups, uint32_t idle_us, uint32_t window_sets, flh_engine** out) {
  if (!out) return fl_set_error(FLH_E_ARG, "null out pointer");
  *out = nullptr;
  int rc = fl_need_init();
  if (rc) return rc;
  // Half as many workers as compute units by default: 128 workers serve 4 MiB batches, two in flight, every 5.9 us and
  // 16 MiB batches every 12.2 us (2.8 and 5.5 TB/s, 4 x bytes); 256 workers 6.1 and 12.7 us, 32 workers 10.1 and 31 us.
  if (workgroups == 0) workgroups = (uint32_t)g_cus / 2 + 1;
  if (window_sets < 1 || window_sets > kEngineDevRing) return fl_set_error(FLH_E_ARG, "an engine rotates 1..%u window sets, not %u", kEngineDevRing, window_sets);
  if (workgroups < 2 || workgroups > 1024) return fl_set_error(FLH_E_ARG, "an engine takes 2..1024 workgroups (a dispatcher and workers), not %u", workgroups);
  flh_engine* e = new (std::nothrow) flh_engine();
  if (!e) return fl_set_error(FLH_E_HIP, "out of host memory");
  memset(e, 0, sizeof(*e));
  e->device = device;
  e->workers = workgroups - 1;
  e->sets = window_sets;
  e->host_slots = 64;
  e->idle_us = idle_us ? idle_us : 200;
  e->wait_us = (uint64_t)g_engine_wait_us;   // two seconds unless a test has asked for less (flh_tune "engine_wait_us")
  e->resident_us = 1000;
  // whatever has been allocated when a call fails goes back through the one cleanup path (which takes null members)
  auto build = [&]() -> int {
    FL_HIP(hipSetDevice(device));
    FL_HIP(hipStreamCreateWithFlags(&e->stream, hipStreamNonBlocking));
    FL_HIP(hipHostMalloc((void**)&e->h_ring, (size_t)e->host_slots * kEngineDescBytes, hipHostMallocMapped));
    FL_HIP(hipHostGetDevicePointer((void**)&e->d_ring_host, e->h_ring, 0));
    FL_HIP(hipHostMalloc((void**)&e->h_ctl, sizeof(EngineHostCtl), hipHostMallocMapped));
    memset(e->h_ctl, 0, sizeof(EngineHostCtl));
    FL_HIP(hipHostGetDevicePointer((void**)&e->d_ctl_host, e->h_ctl, 0));
    FL_HIP(hipMalloc((void**)&e->dev_ring, (size_t)kEngineDevRing * kEngineDescBytes));
    FL_HIP(hipMalloc((void**)&e->dctl, sizeof(EngineDevCtl)));
    FL_HIP(hipMemset(e->dctl, 0, sizeof(EngineDevCtl)));
    if (g_engine_trace) {
      e->trace_slots = 1024;
      FL_HIP(hipMalloc((void**)&e->d_trace, (size_t)e->trace_slots * kEngineStamps * sizeof(uint64_t)));
      FL_HIP(hipMemset(e->d_trace, 0, (size_t)e->trace_slots * kEngineStamps * sizeof(uint64_t)));
    }
    return FLH_OK;
  };
  rc = build();
  if (rc) { (void)flh_engine_destroy(e); return rc; }
  *out = e;
  return FLH_OK;
}

int flh_engine_trace(flh_engine* e, uint64_t first_seq, uint32_t n, uint64_t* stamps_out) {
  if (!e || !stamps_out) return fl_set_error(FLH_E_ARG, "null engine or output");
  if (!e->d_trace) return fl_set_error(FLH_E_STATE, "the engine keeps no trace: set flh_tune(\"engine_trace\", 1) before flh_engine_create");
  if (first_seq == 0 || n == 0 || n > e->trace_slots || first_seq - 1 + n > flh_engine_completed(e) || flh_engine_completed(e) - (first_seq - 1) > e->trace_slots)
    return fl_set_error(FLH_E_ARG, "batches %llu..%llu are not among the last %u complete ones", (unsigned long long)first_seq, (unsigned long long)(first_seq + n - 1), e->trace_slots);
  std::vector<uint64_t> all((size_t)e->trace_slots * kEngineStamps);
  FL_HIP(hipMemcpy(all.data(), e->d_trace, all.size() * sizeof(uint64_t), hipMemcpyDeviceToHost));
  for (uint32_t i = 0; i < n; ++i)
    memcpy(stamps_out + (size_t)i * kEngineStamps, &all[(size_t)((first_seq - 1 + i) & (e->trace_slots - 1)) * kEngineStamps], kEngineStamps * sizeof(uint64_t));
  return FLH_OK;
}

int flh_engine_set_resident(flh_engine* e, uint32_t resident_us) {
  if (!e) return fl_set_error(FLH_E_ARG, "null engine");
  e->resident_us = resident_us;   // read by the next start of the resident kernel
  return FLH_OK;
}

// start the resident kernel with the batch the last one stopped at (the stream orders it behind that one's exit)
static int engine_start(flh_engine* e) {
  if (g_engine_fail_start) return fl_set_error(FLH_E_HIP, "engine launch failed: refused by the engine_fail_start test hook");
  int prev = -1;
  (void)hipGetDevice(&prev);
  if (prev != e->device) FL_HIP(hipSetDevice(e->device));
  struct Back { int dev; ~Back() { if (dev >= 0) (void)hipSetDevice(dev); } } back{prev != e->device ? prev : -1};
  EngineArgs a;
  a.host_ring = e->d_ring_host;
  a.host_slots = e->host_slots;
  a.workers = e->workers;
  a.sets = e->sets;
  a.gen = (uint32_t)(e->launches % 0xfffffffeull) + 1;   // never 0, which is what the quit word holds before any engine has left
  a.hctl = e->d_ctl_host;
  a.dev_ring = e->dev_ring;
  a.dctl = e->dctl;
  a.start = __atomic_load_n(&e->h_ctl->exited_at, __ATOMIC_ACQUIRE);
  a.idle_ticks = e->idle_us * 100;     // the wall clock counts at 100 MHz
  a.wait_ticks = e->wait_us * 100;
  a.resident_ticks = e->resident_us * 100;
  a.inject_fault = g_engine_inject_fault ? 1u : 0u;
  a.trace = e->d_trace;
  a.trace_mask = e->trace_slots ? e->trace_slots - 1 : 0;
  __atomic_store_n(&e->h_ctl->state, 1u, __ATOMIC_RELEASE);
  hipLaunchKernelGGL(fl_engine_kernel, dim3(e->workers + 1), dim3(kCopyBlock), 0, e->stream, a);
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) {
    __atomic_store_n(&e->h_ctl->state, 0u, __ATOMIC_RELEASE);
    return fl_set_error(FLH_E_HIP, "engine launch failed: %s", hipGetErrorString(err));
  }
  e->launches++;
  return FLH_OK;
}

// The engine is down (state 0: the dispatcher has left, and it publishes nothing after that) and never published batch
// `seq`: take the batch back out of the ring, so that no later engine executes it.  Only then may the caller carry it
// some other way.
static void engine_take_back(flh_engine* e, uint64_t seq) {
  e->submitted = seq;
  __atomic_store_n(&e->h_ctl->tail, seq, __ATOMIC_SEQ_CST);
}

static int engine_submit(flh_engine* e, uint32_t kind, const flh_batch_params* b, const flh_windows* win, const flh_windows* landing,
                         flh_chunk_desc* d_table_out, flh_sched_hdr* d_hdr_out, int32_t* d_status, uint64_t* seq_out, uint64_t* seg_base_out) {
  if (!e || !seq_out) return fl_set_error(FLH_E_ARG, "null engine or sequence pointer");
  if (kind > kEngineRecv) return fl_set_error(FLH_E_ARG, "unknown kind of batch %u", kind);
  if ((kind == kEngineSend) != (landing != nullptr)) return fl_set_error(FLH_E_ARG, "landing windows go with FLH_ENGINE_SEND and with nothing else");
  if (__atomic_load_n(&e->h_ctl->error, __ATOMIC_ACQUIRE)) return fl_set_error(FLH_E_STATE, "the engine went down on a wait that ran out");
  // the ring slot must be free: its last occupant complete
  const uint64_t seq = e->submitted;
  if (seq >= e->host_slots && flh_engine_completed(e) + e->host_slots <= seq)
    return fl_set_error(FLH_E_NOMEM, "the engine's descriptor ring is full (%u batches in flight)", e->host_slots);
  BatchPlan pl;
  int rc = plan_batch(b, pl);
  if (rc) return rc;
  if (seg_base_out) memcpy(seg_base_out, pl.seg_base, sizeof(pl.seg_base));
  EngineDesc* d = (EngineDesc*)(e->h_ring + (size_t)(seq % e->host_slots) * kEngineDescBytes);
  flh_uniform_params u = b->u;
  u.total_bytes = (uint64_t)pl.n_chunks * b->u.chunk_bytes;
  u.epoch_bytes = 0;
  u.d_done_word = nullptr;
  u.d_start_word = nullptr;
  u.done_event = nullptr;
  FusedBatchCarryArgs a;
  rc = fill_fused(a, kind == kEngineRecv ? 1 : 0, win, &u, d_table_out, d_hdr_out, d_status, landing);
  if (rc) return rc < 0 ? rc : fl_set_error(FLH_E_ARG, "empty batch");
  memset(&a.carry, 0, sizeof(a.carry));
  if (landing) a.carry = *landing;
  a.total_bytes = b->u.total_bytes;
  a.dest_order = 0;
  a.src_base = 0;
  a.xcd_map = 0;                        // the engine's workers take tiles by their own stride
  a.n_req = b->n_req;
  a.n_seg = pl.n_seg;
  for (uint32_t q = 0; q < FLH_BATCH_MAX; ++q) {
    a.first[q] = pl.first[q];
    a.seg_of[q] = pl.seg_of[q];
    a.req_user[q] = nullptr;
    a.req_bytes[q] = 0;
    a.onward[q] = nullptr;
    if (q >= b->n_req) continue;
    if ((kind != kEngineRecv && !b->d_src[q]) || (kind != kEngineSend && !b->d_dst[q])) return fl_set_error(FLH_E_ARG, "request %u of the batch has no buffer", q);
    a.req_user[q] = kind == kEngineRecv ? (uint8_t*)b->d_dst[q] : (uint8_t*)b->d_src[q];
    a.req_bytes[q] = b->bytes[q];
    if (kind == kEngineLoop) a.onward[q] = (uint8_t*)b->d_dst[q];
  }
  for (uint32_t k = 0; k < FLH_SEG_MAX; ++k) a.seg[k] = pl.seg[k];
  memcpy(&d->a, &a, sizeof(a));
  d->kind = kind;
  d->share = engine_share(a.n_chunks * a.tiles_per_chunk, e->workers);
  d->tiles = (a.n_chunks * a.tiles_per_chunk + d->share - 1) / d->share;
  e->submitted = seq + 1;
  *seq_out = seq + 1;
  // The tail goes out, then the state is read; the dispatcher stores the state, then reads the tail: one of the two
  // sees the other's store, so a batch is never left behind by an engine that is going down.
  __atomic_store_n(&e->h_ctl->tail, seq + 1, __ATOMIC_SEQ_CST);
  __atomic_thread_fence(__ATOMIC_SEQ_CST);
  uint32_t st = __atomic_load_n(&e->h_ctl->state, __ATOMIC_SEQ_CST);
  for (int spin = 0; st == 2 && spin < 4000000; ++spin) st = __atomic_load_n(&e->h_ctl->state, __ATOMIC_ACQUIRE);   // it decides within microseconds
  if (st == 2) {
    // It has not decided (a dispatcher that lost its compute unit to another process's work can take that long).  An
    // error from here on must be final -- the caller then carries the batch some other way, and an engine that woke
    // up later and executed it as well would write into buffers that have since been given away.  So the engine is
    // told to leave and waited for, every wait inside it being bounded; what it did with the batch is then known.
    (void)hipSetDevice(e->device);
    __atomic_store_n(&e->h_ctl->stop, 1u, __ATOMIC_RELEASE);
    const hipError_t err = hipStreamSynchronize(e->stream);
    __atomic_store_n(&e->h_ctl->stop, 0u, __ATOMIC_RELEASE);
    if (err != hipSuccess) return fl_set_error(FLH_E_HIP, "the engine did not go down: %s", hipGetErrorString(err));
    st = __atomic_load_n(&e->h_ctl->state, __ATOMIC_ACQUIRE);
  }
  if (st == 0) {
    // down: either it took the batch with it (published before it left: its workers finish it), or the batch is still
    // in the ring and the next engine starts with it
    if (__atomic_load_n(&e->h_ctl->exited_at, __ATOMIC_ACQUIRE) > seq) return FLH_OK;
    if (__atomic_load_n(&e->h_ctl->error, __ATOMIC_ACQUIRE)) {
      engine_take_back(e, seq);
      return fl_set_error(FLH_E_STATE, "the engine went down on a wait that ran out");
    }
    rc = engine_start(e);
    if (rc) engine_take_back(e, seq);
    return rc;
  }
  return FLH_OK;
}

int flh_engine_submit(flh_engine* e, const flh_batch_params* b, const flh_windows* win, flh_chunk_desc* d_table_out,
                      flh_sched_hdr* d_hdr_out, int32_t* d_status, uint64_t* seq_out, uint64_t* seg_base_out) {
  return engine_submit(e, kEngineLoop, b, win, nullptr, d_table_out, d_hdr_out, d_status, seq_out, seg_base_out);
}

int flh_engine_submit_wire(flh_engine* e, uint32_t kind, const flh_batch_params* b, const flh_windows* win, const flh_windows* landing,
                           flh_chunk_desc* d_table_out, flh_sched_hdr* d_hdr_out, int32_t* d_status, uint64_t* seq_out, uint64_t* seg_base_out) {
  if (kind != kEngineSend && kind != kEngineRecv) return fl_set_error(FLH_E_ARG, "a wire batch is FLH_ENGINE_SEND or FLH_ENGINE_RECV");
  return engine_submit(e, kind, b, win, landing, d_table_out, d_hdr_out, d_status, seq_out, seg_base_out);
}

// An engine that left with batches still in its ring (its time as a resident was up) and that no submit has started
// again since: start it.  Cheap to ask -- two loads of host memory -- when there is nothing to do.
int flh_engine_needs_start(const flh_engine* e) {
  if (!e) return 0;
  if (__atomic_load_n(&e->h_ctl->state, __ATOMIC_ACQUIRE) != 0) return 0;
  return __atomic_load_n(&e->h_ctl->tail, __ATOMIC_ACQUIRE) > __atomic_load_n(&e->h_ctl->exited_at, __ATOMIC_ACQUIRE) &&
         __atomic_load_n(&e->h_ctl->error, __ATOMIC_ACQUIRE) == 0;
}
int flh_engine_poke(flh_engine* e) {
  if (!flh_engine_needs_start(e)) return FLH_OK;
  return engine_start(e);
}

// Batches complete, counted in order: batch c is complete once its ring slot reports it or a later batch of the slot
// (which cannot have started before).  Batches with different workers may finish out of order; the prefix is what a
// caller that reuses window sets and ring slots in order needs.
uint64_t flh_engine_completed(const flh_engine* e) {
  if (!e) return 0;
  uint64_t* known = const_cast<uint64_t*>(&e->completed);
  uint64_t c = __atomic_load_n(known, __ATOMIC_ACQUIRE);   // pairs with the release below: what the thread that moved it forward had acquired from the device
  const uint64_t from = c;
  while (__atomic_load_n(&e->h_ctl->done[c % kEngineDevRing], __ATOMIC_ACQUIRE) >= c + 1) ++c;
  if (c != from) {
    uint64_t seen = from;
    while (seen < c && !__atomic_compare_exchange_n(known, &seen, c, true, __ATOMIC_RELEASE, __ATOMIC_RELAXED)) {}
  }
  return c;
}

int flh_engine_error(const flh_engine* e) {
  return e ? __atomic_load_n(&e->h_ctl->error, __ATOMIC_ACQUIRE) : FLH_E_ARG;
}

uint64_t flh_engine_launches(const flh_engine* e) { return e ? e->launches : 0; }

int flh_engine_destroy(flh_engine* e) {
  if (!e) return FLH_OK;
  (void)hipSetDevice(e->device);
  if (e->h_ctl) __atomic_store_n(&e->h_ctl->stop, 1u, __ATOMIC_RELEASE);
  if (e->stream) (void)hipStreamSynchronize(e->stream);   // the dispatcher sees the flag within a poll
  if (e->h_ring) (void)hipHostFree(e->h_ring);
  if (e->h_ctl) (void)hipHostFree(e->h_ctl);
  if (e->dev_ring) (void)hipFree(e->dev_ring);
  if (e->dctl) (void)hipFree(e->dctl);
  if (e->d_trace) (void)hipFree(e->d_trace);
  if (e->stream) (void)hipStreamDestroy(e->stream);
  delete e;
  return FLH_OK;
}

int flh_copy(void* d_dst, const void* d_src, uint64_t bytes, void* stream) {
  if (bytes == 0) return FLH_OK;
  if (!d_dst || !d_src) return fl_set_error(FLH_E_ARG, "null pointer");
  int rc = fl_need_init();
  if (rc) return rc;
  fl_prof().kid = 6;
  const uint32_t tile = FLH_TILE_BYTES;
  const uint32_t grid = fl_copy_grid((bytes + tile - 1) / tile);
  hipStream_t s = (hipStream_t)stream;
  const uint32_t xcd = grid == (bytes + tile - 1) / tile ? fl_xcd_full(grid) : 0;   // only with one workgroup per tile
  if (fl_use_nt(2 * bytes)) FL_LAUNCH(fl_plain_copy<3>, dim3(grid), dim3(kCopyBlock), 0, s, (uint8_t*)d_dst, (const uint8_t*)d_src, bytes, tile, xcd);
  else FL_LAUNCH(fl_plain_copy<0>, dim3(grid), dim3(kCopyBlock), 0, s, (uint8_t*)d_dst, (const uint8_t*)d_src, bytes, tile, xcd);
  FL_HIP(hipGetLastError());
  return FLH_OK;
}

int flh_copy_runs(void* const* d_dst, const void* const* d_src, const uint64_t* bytes, uint32_t n, void* stream) {
  if (n == 0) return FLH_OK;
  if (!d_dst || !d_src || !bytes) return fl_set_error(FLH_E_ARG, "null pointer");
  if (n > FLH_MAX_LANES) return fl_set_error(FLH_E_ARG, "%u runs: at most %d go into one launch", n, FLH_MAX_LANES);
  int rc = fl_need_init();
  if (rc) return rc;
  CopyRuns a;
  memset(&a, 0, sizeof(a));
  a.tile_bytes = FLH_TILE_BYTES;
  uint64_t tiles = 0, total = 0;
  for (uint32_t r = 0; r < FLH_MAX_LANES; ++r) {
    a.first_tile[r] = (uint32_t)tiles;
    if (r >= n || bytes[r] == 0) continue;
    if (!d_dst[r] || !d_src[r]) return fl_set_error(FLH_E_ARG, "run %u has bytes but no buffer", r);
    a.dst[r] = (uint8_t*)d_dst[r];
    a.src[r] = (const uint8_t*)d_src[r];
    a.bytes[r] = bytes[r];
    tiles += (bytes[r] + a.tile_bytes - 1) / a.tile_bytes;
    total += bytes[r];
    if (tiles > 0x7fffffffull) return fl_set_error(FLH_E_ARG, "too many tiles for one launch");
  }
  a.first_tile[FLH_MAX_LANES] = (uint32_t)tiles;
  if (tiles == 0) return FLH_OK;
  // empty runs share their successor's first tile, so the search lands on the run that owns the tile
  a.xcd = fl_xcd_full((uint32_t)tiles);
  fl_prof().kid = 6;
  hipStream_t s = (hipStream_t)stream;
  if (fl_use_nt(2 * total)) FL_LAUNCH(fl_copy_runs<3>, dim3((uint32_t)tiles), dim3(kCopyBlock), 0, s, a);
  else FL_LAUNCH(fl_copy_runs<0>, dim3((uint32_t)tiles), dim3(kCopyBlock), 0, s, a);
  FL_HIP(hipGetLastError());
  return FLH_OK;
}

}  // extern "C"
