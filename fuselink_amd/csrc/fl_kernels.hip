// fl_kernels.hip -- gfx950 kernels of the FuseLink data path and their C entry points:
//   * fl_schedule_kernel : chunk -> (lane, window offset) table, wavefront prefix scans (DPP)
//   * fl_copy_tiles      : striping (user buffer -> lane windows) and reassembly (windows -> user)
//   * fl_page_tiles      : paged gather / scatter (non-contiguous pages <-> lane windows)
//   * fl_plain_copy      : calibration copy with the same inner loop
// The path is a pure HBM-bound byte mover plus one small integer scan; nothing here contracts, so
// no MFMA.  Wavefronts are 64 wide; all cross-lane traffic in the scheduler is DPP row shifts and
// row broadcasts, LDS is used only to pass per-wave totals between the waves of the one workgroup.
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "fl_internal.h"
#include "fuselink_hip.h"

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

// ------------------------------------------------------------------------------------------------
// scheduler
// ------------------------------------------------------------------------------------------------
constexpr int kRowCache = 32;      // credit rows kept in LDS

struct SchedArgs {
  const uint32_t* sizes;
  uint64_t total_bytes;
  const uint64_t* src_off;
  uint64_t src_base;
  const uint32_t* credits;
  uint64_t quantum;
  flh_sched_state* state;
  flh_chunk_desc* table;
  flh_sched_hdr* hdr;
  uint32_t chunk_bytes;
  uint32_t n;
  uint32_t n_lanes;
  uint32_t n_rows;
  uint32_t epoch_len;
  uint32_t tile_bytes;
  uint32_t mode;
  int32_t quantum_shift;  // >= 0 when quantum is a power of two
  int32_t tile_shift;     // >= 0 when tile_bytes is a power of two
  uint32_t inline_credits[FLH_MAX_LANES];  // the one credit row when credits == nullptr
  flh_chunk_desc* table_by_lane;           // optional second copy of the rows in destination order (uniform kernel only)
};

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

// Credit rows -> inclusive prefixes, four rows per wavefront: a row of at most 16 lanes fills one
// 16-lane DPP row, so four row_shr steps scan it and rows never mix.  `raw` holds the rows in LDS.
// A row without any credit (every lane busy) is replaced by equal credits -- the round robin of the
// static policy -- and marked in zero[].
template <int BT>
__device__ __forceinline__ void credit_row_prefixes(const uint32_t* raw, uint32_t R, uint32_t L, int tid,
                                                    uint64_t (*pfx)[FLH_MAX_LANES], uint32_t* zero) {
  const int lane = tid & (kWave - 1);
  const uint32_t sub = (uint32_t)lane & 15u;
#pragma unroll 1
  for (uint32_t r0 = 0; r0 < R; r0 += BT / 16) {
    const uint32_t r = r0 + (uint32_t)tid / 16u;
    const bool live = r < R && sub < L;
    uint64_t v = live ? raw[r * L + sub] : 0u;
    { uint64_t t = dpp_u64<0x111>(v); if (sub >= 1) v += t; }
    { uint64_t t = dpp_u64<0x112>(v); if (sub >= 2) v += t; }
    { uint64_t t = dpp_u64<0x114>(v); if (sub >= 4) v += t; }
    { uint64_t t = dpp_u64<0x118>(v); if (sub >= 8) v += t; }
    const int top = (lane | 15) << 2;
    const uint32_t wlo = (uint32_t)__builtin_amdgcn_ds_bpermute(top, (int)(uint32_t)v);
    const uint32_t whi = (uint32_t)__builtin_amdgcn_ds_bpermute(top, (int)(uint32_t)(v >> 32));
    const bool none = (wlo | whi) == 0;
    if (none) v = sub + 1;
    if (live) pfx[r][sub] = v;
    if (r < R && sub == 0) zero[r] = none;
  }
}

template <typename T> __device__ __forceinline__ T wave_incl_sum(T v, int lane);
template <> __device__ __forceinline__ uint32_t wave_incl_sum<uint32_t>(uint32_t v, int lane) { return wave_incl_sum_u32(v, lane); }
template <> __device__ __forceinline__ uint64_t wave_incl_sum<uint64_t>(uint64_t v, int lane) { return wave_incl_sum_u64(v, lane); }

// In-wavefront part of the window offsets: for every lane l, scan the threads' bytes on l and hand
// each chunk on l its exclusive position.  Four lanes go through the scan side by side so that their
// DPP chains overlap (a lone wavefront per SIMD has nothing else to hide that latency with).  The
// wavefront's total of lane l is parked in thread l and goes to LDS once at the end.
// T is the width of the partial sums (32 bits when the whole pass moves less than 4 GiB).
template <typename T, int K>
__device__ __forceinline__ void lane_pass(const uint32_t (&s)[K], const uint32_t (&ln)[K], uint32_t L, int lane,
                                          uint64_t* w_lane_row, uint64_t (&off)[K]) {
  constexpr int G = 4;
  uint64_t my_total = 0;
#pragma unroll 1
  for (uint32_t l0 = 0; l0 < L; l0 += G) {
    T v[G], inc[G];
#pragma unroll
    for (int g = 0; g < G; ++g) {
      v[g] = 0;
#pragma unroll
      for (int k = 0; k < K; ++k) v[g] += ln[k] == l0 + g ? (T)s[k] : (T)0;
    }
#pragma unroll
    for (int g = 0; g < G; ++g) inc[g] = wave_incl_sum<T>(v[g], lane);
#pragma unroll
    for (int g = 0; g < G; ++g) {
      uint64_t ex = (uint64_t)(inc[g] - v[g]);
#pragma unroll
      for (int k = 0; k < K; ++k) {
        if (ln[k] == l0 + g) { off[k] = ex; ex += s[k]; }
      }
      const uint64_t tot = sizeof(T) == 8 ? bcast_lane_u64((uint64_t)inc[g], kWave - 1) : (uint64_t)bcast_lane_u32((uint32_t)inc[g], kWave - 1);
      if ((uint32_t)lane == l0 + g) my_total = tot;
    }
  }
  if ((uint32_t)lane < L) w_lane_row[lane] = my_total;
}

// One workgroup of NW wavefronts walks the chunk list in passes of NW*64*K chunks; thread t owns K
// consecutive chunks of a pass.  Per pass: thread-local sums, three wavefront scans (epoch-segmented
// bytes, bytes, tiles), the lane of each chunk from its quantum slot, one wavefront scan per lane
// for the window offsets.  LDS only carries per-wavefront totals and the running lane offsets.
template <int NW, int K>
__global__ __launch_bounds__(NW * kWave) void fl_schedule_kernel(SchedArgs a) {
  constexpr int BT = NW * kWave;
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid / kWave;
  const uint32_t L = a.n_lanes;

  // credit rows as inclusive prefixes; row r occupies rowpfx[r][0..L), W = rowpfx[r][L-1]
  __shared__ uint64_t rowpfx[kRowCache][FLH_MAX_LANES];
  __shared__ uint32_t rowzero[kRowCache];  // the row had no credit at all
  // the same prefixes in 32 bits, entries past L-1 saturated, for rows whose credits sum below 2^32
  __shared__ __attribute__((aligned(16))) uint32_t rowpfx32[kRowCache][FLH_MAX_LANES];
  __shared__ uint32_t rows_wide;  // some row sums to 2^32 or more: use the 64-bit prefixes
  __shared__ uint64_t w_seg_v[NW];
  __shared__ uint32_t w_seg_f[NW];
  __shared__ uint64_t w_run[NW];
  __shared__ uint32_t w_tiles[NW];
  __shared__ uint64_t w_lane[NW][FLH_MAX_LANES];  // per-wavefront lane totals, then absolute bases
  __shared__ uint64_t lane_off[FLH_MAX_LANES];    // next free byte of every window
  __shared__ uint64_t lane_off0[FLH_MAX_LANES];
  __shared__ uint32_t cnt_lane[FLH_MAX_LANES];
  __shared__ uint32_t sh_flags;

  // One wavefront per row: lanes 0..L-1 load the row in a single access, a scan forms the prefixes.
  // A row without any credit (every lane busy) is replaced by equal credits -- the round-robin of
  // the static policy -- and flagged.
  const bool rows_cached = a.n_rows <= (uint32_t)kRowCache;
  uint32_t flags = 0;
  __shared__ uint32_t raw[kRowCache * FLH_MAX_LANES];
  if (rows_cached) {
    // all credit rows in one round trip to memory, then one wavefront scan per row out of LDS
    for (uint32_t e = tid; e < a.n_rows * L; e += BT) raw[e] = a.credits ? a.credits[e] : a.inline_credits[e];
  }
  // the carried state and the first pass's sizes are requested before anything waits on the credit rows,
  // so that the kernel pays one round trip to memory, not three in a row
  uint64_t k0 = 0, p_carry = 0, run_carry = 0;  // carried state, identical in every thread
  uint32_t tiles_carry = 0;
  if (a.state) {
    k0 = a.state->chunk_index;
    if (!(a.mode & FLH_SCHED_NEW_EPOCH)) p_carry = a.state->epoch_bytes;
  }
  uint64_t off_in = 0;
  if (tid < FLH_MAX_LANES && a.state && !(a.mode & FLH_SCHED_RESET_OFFSETS)) off_in = a.state->lane_off[tid];
  uint32_t s_next[K];
#pragma unroll
  for (int k = 0; k < K; ++k) {
    const uint32_t i = (uint32_t)tid * K + k;
    s_next[k] = (a.sizes && i < a.n) ? a.sizes[i] : 0;
  }
  if (rows_cached) {
    __syncthreads();
    credit_row_prefixes<BT>(raw, a.n_rows, L, tid, rowpfx, rowzero);
    if (tid == 0) rows_wide = 0;
    __syncthreads();
    for (uint32_t e = tid; e < a.n_rows * FLH_MAX_LANES; e += BT) {
      const uint32_t r = e / FLH_MAX_LANES, l = e % FLH_MAX_LANES;
      const uint64_t v = l + 1 < L ? rowpfx[r][l] : ~0ull;  // the last prefix is W > slot: never counted
      rowpfx32[r][l] = v >> 32 ? 0xffffffffu : (uint32_t)v;
      if (l == L - 1 && (rowpfx[r][l] >> 32)) rows_wide = 1;
    }
  }
  if (tid < FLH_MAX_LANES) {
    const uint64_t o = off_in;
    lane_off[tid] = o;
    lane_off0[tid] = o;
    cnt_lane[tid] = 0;
  }
  if (tid == 0) sh_flags = 0;
  __syncthreads();

  const bool wide = rows_cached && rows_wide != 0;
#pragma unroll 1
  for (uint32_t pass = 0; pass < a.n; pass += BT * K) {
    const uint32_t i0 = pass + (uint32_t)tid * K;
    uint32_t s[K], tl[K], row[K], ep[K], ln[K];
    bool head[K];
    // ---- epoch, position in epoch and credit row of my first chunk; the rest follow by counting ----
    uint64_t e_cur = 0;
    uint32_t pos = 0, r_cur = 0;
    if (a.epoch_len) {
      const uint64_t g0 = k0 + i0;
      e_cur = div_u64(g0, a.epoch_len);
      pos = (uint32_t)(g0 - e_cur * a.epoch_len);
      r_cur = (uint32_t)mod_u64(e_cur, a.n_rows);
    }
    // ---- load sizes, mark epoch heads, thread-local aggregates -----------------------------------
    uint64_t seg_v = 0;
    uint32_t seg_f = 0;
    uint64_t run = 0;
    uint32_t tiles = 0;
#pragma unroll
    for (int k = 0; k < K; ++k) {
      const uint32_t i = i0 + k;
      uint32_t sz = 0;
      bool hd = false;
      if (i < a.n) {
        if (a.sizes) {
          sz = s_next[k];
        } else {
          const uint64_t o = (uint64_t)i * a.chunk_bytes;
          const uint64_t rem = o < a.total_bytes ? a.total_bytes - o : 0;
          sz = (uint32_t)(rem < a.chunk_bytes ? rem : a.chunk_bytes);
        }
        hd = a.epoch_len && pos == 0;
      }
      s[k] = sz;
      head[k] = hd;
      row[k] = r_cur;
      ep[k] = (uint32_t)e_cur;
      tl[k] = a.tile_shift >= 0 ? (sz + a.tile_bytes - 1) >> a.tile_shift : (sz + a.tile_bytes - 1) / a.tile_bytes;
      if (hd) { seg_v = 0; seg_f = 1; }
      seg_v += sz;
      run += sz;
      tiles += tl[k];
      if (a.epoch_len && ++pos == a.epoch_len) {
        pos = 0;
        ++e_cur;
        if (++r_cur == a.n_rows) r_cur = 0;
      }
    }
    if (a.sizes) {  // next pass's sizes travel while this pass computes
#pragma unroll
      for (int k = 0; k < K; ++k) {
        const uint64_t i = (uint64_t)i0 + (uint64_t)BT * K + k;
        s_next[k] = i < a.n ? a.sizes[i] : 0;
      }
    }
    // ---- block-wide exclusive prefixes of (segmented bytes, bytes, tiles) --------------------------
    uint64_t sv = seg_v;
    uint32_t sf = seg_f;
    wave_incl_segsum_u64(sv, sf, lane);
    const uint64_t run_incl = wave_incl_sum_u64(run, lane);
    const uint32_t tiles_incl = wave_incl_sum_u32(tiles, lane);
    uint64_t seg_ex_v = wave_shift_up_u64(sv, lane);
    uint32_t seg_ex_f = wave_shift_up_u32(sf, lane);
    uint64_t run_ex = run_incl - run;
    uint32_t tiles_ex = tiles_incl - tiles;
    if (lane == kWave - 1) { w_seg_v[wave] = sv; w_seg_f[wave] = sf; w_run[wave] = run_incl; w_tiles[wave] = tiles_incl; }
    __syncthreads();
    uint64_t tot_seg_v = 0, tot_run = 0;
    uint32_t tot_seg_f = 0, tot_tiles = 0;
    {
      uint64_t pv = 0, pr = 0;
      uint32_t pf = 0, pt = 0;
#pragma unroll
      for (int w = 0; w < NW; ++w) {
        if (w == wave) { pv = tot_seg_v; pf = tot_seg_f; pr = tot_run; pt = tot_tiles; }
        const uint64_t wv = w_seg_v[w];
        const uint32_t wf = w_seg_f[w];
        tot_seg_v = wf ? wv : tot_seg_v + wv;
        tot_seg_f |= wf;
        tot_run += w_run[w];
        tot_tiles += w_tiles[w];
      }
      // combine the earlier wavefronts' aggregate with my in-wavefront exclusive value
      if (!seg_ex_f) seg_ex_v += pv;
      seg_ex_f |= pf;
      run_ex += pr;
      tiles_ex += pt;
    }
    // bytes of my epoch before my first chunk
    uint64_t P = seg_ex_f ? seg_ex_v : p_carry + seg_ex_v;

    // ---- lane of each chunk ------------------------------------------------------------------------------
#pragma unroll
    for (int k = 0; k < K; ++k) {
      const uint32_t i = i0 + k;
      ln[k] = FLH_MAX_LANES;  // matches no lane: chunks past the end count nowhere
      if (i < a.n) {
        if (head[k]) P = 0;
        const uint32_t r = row[k];
        uint64_t W;
        bool equal = false;  // no lane has credit: equal credits stand in
        if (rows_cached) {
          W = rowpfx[r][L - 1];
          if (rowzero[r]) flags |= FLH_SCHED_F_NO_CREDIT;
        } else {
          W = 0;
#pragma unroll 1
          for (uint32_t l = 0; l < L; ++l) W += a.credits[(size_t)r * L + l];
          if (W == 0) { W = L; equal = true; flags |= FLH_SCHED_F_NO_CREDIT; }
        }
        const uint64_t qn = a.quantum_shift >= 0 ? (P >> a.quantum_shift) : div_u64(P, a.quantum);
        const uint64_t slot = mod_u64(qn, W);
        // lane = number of inclusive prefixes <= slot (zero-credit lanes repeat the prefix and are skipped)
        uint32_t pick = 0;
        if (rows_cached && !wide) {
          const uint32_t slot32 = (uint32_t)slot;  // slot < W < 2^32
          const u32x4* pr = reinterpret_cast<const u32x4*>(rowpfx32[r]);
          const u32x4 p0 = pr[0], p1 = pr[1], p2 = pr[2], p3 = pr[3];
          pick = (p0.x <= slot32) + (p0.y <= slot32) + (p0.z <= slot32) + (p0.w <= slot32) + (p1.x <= slot32) + (p1.y <= slot32) +
                 (p1.z <= slot32) + (p1.w <= slot32) + (p2.x <= slot32) + (p2.y <= slot32) + (p2.z <= slot32) + (p2.w <= slot32) +
                 (p3.x <= slot32) + (p3.y <= slot32) + (p3.z <= slot32) + (p3.w <= slot32);
        } else if (rows_cached) {
#pragma unroll 1
          for (uint32_t l = 0; l + 1 < L; ++l) pick += rowpfx[r][l] <= slot;
        } else if (equal) {
          pick = (uint32_t)slot;
        } else {
          uint64_t kk = 0;
#pragma unroll 1
          for (uint32_t l = 0; l + 1 < L; ++l) { kk += a.credits[(size_t)r * L + l]; pick += kk <= slot; }
        }
        ln[k] = pick;
        atomicAdd(&cnt_lane[pick], 1u);  // LDS counter of chunks per lane
        P += s[k];
      }
    }
    // ---- window offsets: in-wavefront scans per lane, then wavefront bases through LDS -----------------
    uint64_t off[K];
#pragma unroll
    for (int k = 0; k < K; ++k) off[k] = 0;
    if ((tot_run >> 32) == 0) lane_pass<uint32_t, K>(s, ln, L, lane, w_lane[wave], off);
    else lane_pass<uint64_t, K>(s, ln, L, lane, w_lane[wave], off);
    __syncthreads();
    if ((uint32_t)tid < L) {
      uint64_t at = lane_off[tid];
#pragma unroll
      for (int w = 0; w < NW; ++w) {
        const uint64_t x = w_lane[w][tid];
        w_lane[w][tid] = at;
        at += x;
      }
      lane_off[tid] = at;
    }
    __syncthreads();
    // ---- emit rows ---------------------------------------------------------------------------------------
    uint64_t run_i = run_carry + run_ex;
    uint32_t tiles_i = tiles_carry + tiles_ex;
#pragma unroll
    for (int k = 0; k < K; ++k) {
      const uint32_t i = i0 + k;
      if (i < a.n) {
        flh_chunk_desc d;
        d.src_off = a.src_off ? a.src_off[i] : a.src_base + run_i;
        d.win_off = (a.mode & FLH_SCHED_MIRROR) ? d.src_off : w_lane[wave][ln[k]] + off[k];
        d.len = s[k];
        d.lane = ln[k];
        d.tile_base = tiles_i;
        d.epoch = ep[k];
        a.table[i] = d;
        run_i += s[k];
        tiles_i += tl[k];
      }
    }
    // ---- carries -------------------------------------------------------------------------------------------
    p_carry = tot_seg_f ? tot_seg_v : p_carry + tot_seg_v;
    run_carry += tot_run;
    tiles_carry += tot_tiles;
  }

  // ---- header and state --------------------------------------------------------------------------------------
  if (__builtin_amdgcn_ballot_w64(flags != 0) && lane == 0) atomicOr(&sh_flags, FLH_SCHED_F_NO_CREDIT);
  __syncthreads();
  if (tid < FLH_MAX_LANES) {
    a.hdr->lane_bytes[tid] = lane_off[tid] - lane_off0[tid];
    a.hdr->lane_chunks[tid] = cnt_lane[tid];
    if (a.state) a.state->lane_off[tid] = lane_off[tid];
  }
  if (tid == 0) {
    a.hdr->total_bytes = run_carry;
    a.hdr->total_tiles = tiles_carry;
    a.hdr->n_chunks = a.n;
    a.hdr->flags = sh_flags;
    a.hdr->uniform_tiles = (!a.sizes && a.n) ? (a.chunk_bytes + a.tile_bytes - 1) / a.tile_bytes : 0;
    if (a.state) {
      a.state->epoch_bytes = p_carry;
      a.state->chunk_index = k0 + a.n;
    }
  }
}

// ------------------------------------------------------------------------------------------------
// scheduler, uniform split
// ------------------------------------------------------------------------------------------------
// When every chunk has the quantum's size (the ordinary message split: sizes == nullptr and
// quantum == chunk_bytes; only the last chunk may be short) the byte prefix of chunk j of an epoch
// is j quanta, so its slot is j mod W and nothing has to be scanned: the number of earlier chunks
// on a lane is a closed form in j,
//     cnt(row, l, x) = #{ y < x : slot y belongs to lane l } = (x / W) * c_l + clamp(x mod W - K_l, 0, c_l),
// whole epochs contribute cnt(row, l, E), and because rows repeat with period R those contributions
// sum in closed form too.  Every chunk is independent, so the table is filled by as many workgroups
// as it takes; the results are identical to the scan kernel's.
struct UniTables {
  uint64_t pfx[kRowCache][FLH_MAX_LANES];   // inclusive credit prefixes (equal credits for an empty row)
  uint64_t pf[kRowCache + 1][FLH_MAX_LANES];  // pf[r][l] = chunks on lane l in whole epochs of rows < r; pf[R] = one period
  uint32_t zero[kRowCache];
};

__device__ __forceinline__ uint64_t uni_cnt(const UniTables& t, uint32_t r, uint32_t l, uint32_t L, uint64_t x) {
  const uint64_t W = t.pfx[r][L - 1];
  const uint64_t hi = t.pfx[r][l];
  const uint64_t K = l ? t.pfx[r][l - 1] : 0;
  const uint64_t c = hi - K;
  const uint64_t full = div_u64(x, W);
  const uint64_t rem = x - full * W;
  const uint64_t part = rem <= K ? 0 : (rem - K < c ? rem - K : c);
  return full * c + part;
}

__device__ __forceinline__ uint32_t uni_lane(const UniTables& t, uint32_t r, uint32_t L, uint64_t j) {
  const uint64_t slot = mod_u64(j, t.pfx[r][L - 1]);
  uint32_t pick = 0;
#pragma unroll 1
  for (uint32_t l = 0; l + 1 < L; ++l) pick += t.pfx[r][l] <= slot;
  return pick;
}

struct UniCtx {
  uint64_t k0, a0, e0, C;
  uint32_t pos0, E, R, L;
};

// chunks of this call, before local index i (0 <= i <= n), that sit on lane l; also returns the lane
// of chunk i itself through *lane_of_i when asked (l == 0xffffffff means "use chunk i's own lane")
__device__ __forceinline__ uint64_t uni_before(const UniTables& t, const UniCtx& c, uint64_t i, uint32_t l, uint32_t* lane_of_i,
                                               uint64_t* epoch_of_i) {
  if (c.E == 0) {
    const uint64_t j = c.a0 + i;
    if (lane_of_i) { *lane_of_i = uni_lane(t, 0, c.L, j); if (l == 0xffffffffu) l = *lane_of_i; }
    if (epoch_of_i) *epoch_of_i = 0;
    return uni_cnt(t, 0, l, c.L, j) - uni_cnt(t, 0, l, c.L, c.a0);
  }
  const uint64_t g = c.k0 + i;
  const uint64_t e = div_u64(g, c.E);
  const uint64_t pos = g - e * c.E;
  const uint32_t r = (uint32_t)mod_u64(e, c.R);
  if (epoch_of_i) *epoch_of_i = e;
  if (e == c.e0) {
    const uint64_t j = c.a0 + (pos - c.pos0);
    if (lane_of_i) { *lane_of_i = uni_lane(t, r, c.L, j); if (l == 0xffffffffu) l = *lane_of_i; }
    return uni_cnt(t, r, l, c.L, j) - uni_cnt(t, r, l, c.L, c.a0);
  }
  if (lane_of_i) { *lane_of_i = uni_lane(t, r, c.L, pos); if (l == 0xffffffffu) l = *lane_of_i; }
  const uint32_t r0 = (uint32_t)mod_u64(c.e0, c.R);
  const uint64_t m0 = c.E - c.pos0;  // chunks of this call in its first epoch
  uint64_t before = uni_cnt(t, r0, l, c.L, c.a0 + m0) - uni_cnt(t, r0, l, c.L, c.a0);
  // whole epochs e0+1 .. e-1: G(e) - G(e0+1), G(z) = (z / R) * period + pf[z mod R]
  const uint64_t z1 = e, z0 = c.e0 + 1;
  const uint64_t q1 = div_u64(z1, c.R), q0 = div_u64(z0, c.R);
  before += q1 * t.pf[c.R][l] + t.pf[z1 - q1 * c.R][l];
  before -= q0 * t.pf[c.R][l] + t.pf[z0 - q0 * c.R][l];
  before += uni_cnt(t, r, l, c.L, pos);
  return before;
}

constexpr int kUniBlock = 256;

// MODE 0: fill the table; the last workgroup also writes the header and, if the grid is a single
//         workgroup, the state (in place: every read of the old state precedes the barrier).
// MODE 1: write the state only (second launch after a multi-workgroup MODE 0, so that no workgroup
//         can still be reading the old state).
template <int MODE>
__global__ __launch_bounds__(kUniBlock) void fl_schedule_uniform_kernel(SchedArgs a) {
  __shared__ UniTables t;
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid / kWave;
  const uint32_t L = a.n_lanes, R = a.n_rows;
  // all credit rows in one round trip to memory, then one wavefront scan per row out of LDS
  __shared__ uint32_t raw[kRowCache * FLH_MAX_LANES];
  for (uint32_t e = tid; e < R * L; e += kUniBlock) raw[e] = a.credits ? a.credits[e] : a.inline_credits[e];
  // the carried state is requested before anything waits on the credit rows
  const uint64_t k0_in = a.state ? a.state->chunk_index : 0;
  const uint64_t p0 = (a.state && !(a.mode & FLH_SCHED_NEW_EPOCH)) ? a.state->epoch_bytes : 0;
  __syncthreads();
  credit_row_prefixes<kUniBlock>(raw, R, L, tid, t.pfx, t.zero);
  __syncthreads();
  // chunks per lane of one whole epoch under each row (all rows at once), then prefixed over the rows
  for (uint32_t e = tid; e < R * L; e += kUniBlock) {
    const uint32_t r = e / L, l = e - r * L;
    t.pf[r + 1][l] = a.epoch_len ? uni_cnt(t, r, l, L, a.epoch_len) : 0;
  }
  __syncthreads();
  if ((uint32_t)tid < L) {
    uint64_t run = 0;
#pragma unroll 1
    for (uint32_t r = 0; r < R; ++r) {
      const uint64_t x = t.pf[r + 1][tid];
      t.pf[r][tid] = run;
      run += x;
    }
    t.pf[R][tid] = run;
  }
  __syncthreads();

  UniCtx c;
  c.C = a.chunk_bytes;
  c.E = a.epoch_len;
  c.R = R;
  c.L = L;
  c.k0 = k0_in;
  c.e0 = c.E ? div_u64(c.k0, c.E) : 0;
  c.pos0 = c.E ? (uint32_t)(c.k0 - c.e0 * c.E) : 0;
  // quanta already behind the first chunk inside its epoch; an epoch head starts from zero
  c.a0 = (c.E && c.pos0 == 0) ? 0 : div_u64(p0, c.C);
  const bool keep_off = a.state && !(a.mode & FLH_SCHED_RESET_OFFSETS);
  const uint32_t tpc = a.tile_shift >= 0 ? (a.chunk_bytes + a.tile_bytes - 1) >> a.tile_shift : (a.chunk_bytes + a.tile_bytes - 1) / a.tile_bytes;

  // Destination order: rows grouped by lane, the last chunk's lane last (so that a short final chunk stays the
  // final row).  Every workgroup works out where each lane's group starts from the per-lane chunk totals.
  __shared__ uint64_t lane_first[FLH_MAX_LANES];
  __shared__ uint32_t sh_lane_last;
  if (MODE == 0 && a.table_by_lane) {
    if ((uint32_t)tid < L) lane_first[tid] = uni_before(t, c, a.n, (uint32_t)tid, nullptr, nullptr);
    if (tid == kWave) {  // another wavefront than the one busy with the totals
      uint32_t ll;
      (void)uni_before(t, c, a.n - 1, 0xffffffffu, &ll, nullptr);
      sh_lane_last = ll;
    }
    __syncthreads();
    if (tid == 0) {
      uint64_t run = 0;
      uint32_t l = sh_lane_last;
#pragma unroll 1
      for (uint32_t k = 0; k < L; ++k) {
        l = l + 1 == L ? 0 : l + 1;
        const uint64_t x = lane_first[l];
        lane_first[l] = run;
        run += x;
      }
    }
    __syncthreads();
  }

  if (MODE == 0) {
    const uint32_t i = blockIdx.x * kUniBlock + tid;
    if (i < a.n) {
      uint32_t ln;
      uint64_t ep;
      const uint64_t before = uni_before(t, c, i, 0xffffffffu, &ln, &ep);
      const uint64_t o = (uint64_t)i * c.C;
      const uint64_t rem = a.total_bytes - o;
      flh_chunk_desc d;
      d.src_off = a.src_base + o;
      d.win_off = (a.mode & FLH_SCHED_MIRROR) ? d.src_off : (keep_off ? a.state->lane_off[ln] : 0) + before * c.C;
      d.len = (uint32_t)(rem < c.C ? rem : c.C);
      d.lane = ln;
      d.tile_base = i * tpc;
      d.epoch = (uint32_t)ep;
      a.table[i] = d;
      if (a.table_by_lane) {
        const uint64_t pos = lane_first[ln] + before;
        d.tile_base = (uint32_t)pos * tpc;
        a.table_by_lane[pos] = d;
      }
    }
    if (blockIdx.x != gridDim.x - 1) return;
  }
  const bool write_hdr = MODE == 0;
  const bool write_state = a.state && (MODE == 1 || gridDim.x == 1);
  const uint64_t last = a.n - 1;
  const uint64_t len_last = a.total_bytes - last * c.C;
  uint32_t lane_last;
  uint64_t ep_last;
  (void)uni_before(t, c, last, 0xffffffffu, &lane_last, &ep_last);
  uint64_t chunks = 0, bytes = 0, off_in = 0;
  if ((uint32_t)tid < L) {
    chunks = uni_before(t, c, a.n, (uint32_t)tid, nullptr, nullptr);
    bytes = chunks * c.C - ((uint32_t)tid == lane_last ? c.C - len_last : 0);
  }
  if (tid < FLH_MAX_LANES && keep_off) off_in = a.state->lane_off[tid];
  __syncthreads();  // the old state has been read by everyone who needs it
  if (tid < FLH_MAX_LANES) {
    if (write_hdr) {
      a.hdr->lane_bytes[tid] = bytes;
      a.hdr->lane_chunks[tid] = (uint32_t)chunks;
    }
    if (write_state) a.state->lane_off[tid] = off_in + bytes;
  }
  if (tid == 0) {
    if (write_hdr) {
      uint32_t flags = 0;
      const uint64_t n_ep = ep_last - c.e0 + 1;
      const uint32_t look = n_ep < R ? (uint32_t)n_ep : R;
      for (uint32_t k = 0; k < look; ++k) flags |= t.zero[(uint32_t)mod_u64(c.e0 + k, R)] ? FLH_SCHED_F_NO_CREDIT : 0;
      a.hdr->total_bytes = a.total_bytes;
      a.hdr->total_tiles = (uint32_t)last * tpc + (uint32_t)((len_last + a.tile_bytes - 1) / a.tile_bytes);
      a.hdr->n_chunks = a.n;
      a.hdr->flags = flags;
      a.hdr->uniform_tiles = tpc;
    }
    if (write_state) {
      uint64_t p_end;
      if (c.E == 0 || ep_last == c.e0) {
        p_end = ((c.E && c.pos0 == 0) ? 0 : p0) + a.total_bytes;
      } else {
        const uint64_t pos_last = (c.k0 + last) - ep_last * c.E;
        p_end = pos_last * c.C + len_last;
      }
      a.state->epoch_bytes = p_end;
      a.state->chunk_index = c.k0 + a.n;
    }
  }
}

// ------------------------------------------------------------------------------------------------
// copy kernels
// ------------------------------------------------------------------------------------------------

constexpr int kCopyBlock = 256;
constexpr int kCopyUnroll = 8;

template <bool NT>
__device__ __forceinline__ u32x4 ld16(const u32x4* p) {
  return NT ? __builtin_nontemporal_load(p) : *p;
}
template <bool NT>
__device__ __forceinline__ void st16(u32x4* p, u32x4 v) {
  if (NT) __builtin_nontemporal_store(v, p); else *p = v;
}

template <bool NT, int U>
__device__ __forceinline__ void copy_exact(u32x4* __restrict__ d, const u32x4* __restrict__ s, uint32_t tid) {
  u32x4 r[U];
#pragma unroll
  for (int j = 0; j < U; ++j) r[j] = ld16<NT>(s + j * kCopyBlock + tid);
#pragma unroll
  for (int j = 0; j < U; ++j) st16<NT>(d + j * kCopyBlock + tid, r[j]);
}

// Copies `bytes` from src to dst with the whole workgroup.  Fast path: both 16-byte aligned ->
// dwordx4 loads batched kCopyUnroll deep before the stores.  Equal misalignment: byte head up to
// the boundary, vectors, byte tail.  Different misalignment: byte copy (correct, not fast).
template <bool NT>
__device__ __forceinline__ void block_copy(uint8_t* __restrict__ dst, const uint8_t* __restrict__ src,
                                           uint32_t bytes) {
  const uint32_t tid = threadIdx.x;
  const uintptr_t sa = (uintptr_t)src, da = (uintptr_t)dst;
  if (((sa ^ da) & 15) != 0) {
    for (uint32_t i = tid; i < bytes; i += kCopyBlock) dst[i] = src[i];
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
template <int DIR, bool NT>
__global__ __launch_bounds__(kCopyBlock) void fl_copy_tiles(CopyArgs a) {
  const uint32_t total = a.has_hint ? a.hint_total_tiles : a.hdr->total_tiles;
  const uint32_t uniform_tiles = a.has_hint ? a.hint_uniform_tiles : a.hdr->uniform_tiles;
  uint32_t n = a.has_hint ? a.hint_n_chunks : a.hdr->n_chunks;
  if (n > a.n_chunks_max) n = a.n_chunks_max;
  if (n == 0) return;
  for (uint32_t t = blockIdx.x; t < total; t += gridDim.x) {
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

// Uniform split with the header known on the host: a two-dimensional grid (tile in chunk, chunk)
// names the work directly, so a workgroup's only dependent access before its data is the one scalar
// load of its table row.
template <int DIR, bool NT>
__global__ __launch_bounds__(kCopyBlock) void fl_copy_uniform(CopyArgs a) {
  const uint32_t c = blockIdx.y;
  if (c >= a.hint_n_chunks) return;
  const flh_chunk_desc d = a.table[c];
  const uint64_t off = (uint64_t)blockIdx.x * a.tile_bytes;
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
  uint32_t fast;
  uint64_t magic;
  uint32_t cnt0[FLH_MAX_LANES];
};

// Several requests as one message: chunk c belongs to the request r with first[r] <= c < first[r+1];
// its bytes live at user[r] + (c - first[r]) * chunk_bytes.
struct FusedBatchArgs : FusedArgs {
  uint32_t n_req;
  uint32_t first[FLH_BATCH_MAX];   // first chunk of each request
  uint8_t* req_user[FLH_BATCH_MAX];
  uint64_t req_bytes[FLH_BATCH_MAX];
};
template <class A> struct is_batch { static constexpr bool value = false; };
template <> struct is_batch<FusedBatchArgs> { static constexpr bool value = true; };

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

template <int DIR, bool NT, class Args>
__global__ __launch_bounds__(kCopyBlock) void fl_copy_uniform_fused(Args a) {
  constexpr bool BATCH = is_batch<Args>::value;
  if (blockIdx.y >= a.n_chunks) return;
  FusedRow r;
  fused_row(a, r);
  uint32_t c = blockIdx.y, lane = 0;
  uint64_t K = 0, hi = r.pfx[0], before;
  if (DIR == 0 && a.dest_order) {
    // blockIdx.y = k-th chunk in destination order: find the lane whose group holds k, then invert the
    // closed form -- the j-th slot of a lane with credit c_l and first slot K_l is (j / c_l) * W + K_l + j mod c_l.
    const uint64_t x0 = a.quanta_before, x1 = a.quanta_before + a.n_chunks;
    const uint64_t f0 = div_u64(x0, r.W), f1 = div_u64(x1, r.W);
    const uint64_t r0 = x0 - f0 * r.W, r1 = x1 - f1 * r.W;
    uint64_t k = blockIdx.y, cnt0 = 0;
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
    const uint32_t full = (uint32_t)__umul64hi((uint64_t)j, a.magic);  // j / W
    const uint32_t slot = j - full * (uint32_t)r.W;
    uint32_t c0 = a.cnt0[0];
#pragma unroll
    for (int l = 0; l + 1 < FLH_MAX_LANES; ++l) {
      if ((uint32_t)(l + 1) < a.n_lanes && r.pfx[l] <= slot) { lane = l + 1; K = r.pfx[l]; hi = r.pfx[l + 1]; c0 = a.cnt0[l + 1]; }
    }
    before = (uint64_t)full * (hi - K) + (slot - K) - c0;  // slot lies inside the lane's span [K, hi)
  } else {
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
  const uint32_t len = (uint32_t)(rem < a.chunk_bytes ? rem : a.chunk_bytes);
  const uint64_t src_off = a.src_base + chunk_off;
  const uint64_t win_off = before * a.chunk_bytes;
  // where the chunk's bytes live on the user side: in the one buffer, or in its request's buffer
  uint8_t* user = a.user;
  uint64_t user_off = src_off, user_bytes = a.user_bytes;
  if constexpr (BATCH) {
    uint32_t first = 0;
    user = a.req_user[0];
    user_bytes = a.req_bytes[0];
#pragma unroll
    for (int q = 1; q < FLH_BATCH_MAX; ++q) {
      if ((uint32_t)q < a.n_req && a.first[q] <= c) { first = a.first[q]; user = a.req_user[q]; user_bytes = a.req_bytes[q]; }
    }
    user_off = (uint64_t)(c - first) * a.chunk_bytes;
  }

  if (DIR == 0 && blockIdx.x == 0 && threadIdx.x == 0 && a.table) {
    flh_chunk_desc d;
    d.src_off = src_off;
    d.win_off = win_off;
    d.len = len;
    d.lane = lane;
    d.tile_base = c * a.tiles_per_chunk;
    d.epoch = 0;
    a.table[c] = d;
  }
  if (DIR == 0 && blockIdx.x == 0 && blockIdx.y == 0 && a.hdr) {  // header: per-lane totals in closed form
    const uint32_t t = threadIdx.x;
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
      a.hdr->lane_bytes[t] = bytes;
      a.hdr->lane_chunks[t] = (uint32_t)chunks;
    }
    if (t == 0) {
      a.hdr->total_bytes = a.total_bytes;
      a.hdr->total_tiles = (uint32_t)last * a.tiles_per_chunk + (uint32_t)((len_last + a.tile_bytes - 1) / a.tile_bytes);
      a.hdr->n_chunks = a.n_chunks;
      a.hdr->flags = r.zero ? FLH_SCHED_F_NO_CREDIT : 0;
      a.hdr->uniform_tiles = a.tiles_per_chunk;
    }
  }

  const uint64_t off = (uint64_t)blockIdx.x * a.tile_bytes;
  if (off >= len) return;
  const uint32_t bytes = (uint32_t)((len - off) < a.tile_bytes ? (len - off) : a.tile_bytes);
  if (win_off + len > a.win.cap[lane] || user_off + len > user_bytes) {
    if (threadIdx.x == 0) *a.status = FLH_E_RANGE;
    return;
  }
  uint8_t* u = user + user_off + off;
  uint8_t* w = (uint8_t*)a.win.base[lane] + win_off + off;
  if (DIR == 0) block_copy<NT>(w, u, bytes); else block_copy<NT>(u, w, bytes);
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
};

constexpr uint32_t kLdsStage = 16384;

// DIR 0: pool pages -> windows (gather).  DIR 1: windows -> pool pages (scatter).
// LDS: stage each sub-tile through LDS (coalesced global->LDS, barrier, LDS->global).
template <int DIR, bool LDS, bool NT>
__global__ __launch_bounds__(kCopyBlock) void fl_page_tiles(PageArgs a) {
  __shared__ u32x4 stage[LDS ? kLdsStage / 16 : 1];
  const uint64_t total = (uint64_t)a.n_chunks * a.pages_per_chunk * a.subs_per_page;
  for (uint64_t t = blockIdx.x; t < total; t += gridDim.x) {
    const uint32_t sub = (uint32_t)(t % a.subs_per_page);
    const uint64_t rp = t / a.subs_per_page;         // row-major page counter
    const uint32_t c = (uint32_t)(rp / a.pages_per_chunk);
    const uint32_t k = (uint32_t)(rp % a.pages_per_chunk);
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

template <bool NT>
__global__ __launch_bounds__(kCopyBlock) void fl_plain_copy(uint8_t* dst, const uint8_t* src, uint64_t bytes,
                                                            uint32_t tile_bytes) {
  const uint64_t tiles = (bytes + tile_bytes - 1) / tile_bytes;
  for (uint64_t t = blockIdx.x; t < tiles; t += gridDim.x) {
    const uint64_t off = t * tile_bytes;
    const uint32_t len = (uint32_t)((bytes - off) < tile_bytes ? (bytes - off) : tile_bytes);
    block_copy<NT>(dst + off, src + off, len);
  }
}

// ------------------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------------------
thread_local char g_err[512] = "";
int g_device = -1;
int g_cus = 0;
// launch tunables (overridable through NCCL_FUSELINK_* for experiments)
int g_grid_per_cu = 0;     // 0: one workgroup per tile (up to 2^20)
constexpr uint64_t kCacheResidentBytes = 512ull << 20;  // working sets up to this stay largely in the 256 MB Infinity Cache
int g_dest_order = -1;    // fused striping in destination order: -1 = when the working set exceeds the cache, 0 / 1 force
int g_fused_fast = 1;     // host-prepared reciprocal for the fused kernels' slot arithmetic (0 = always divide in the kernel)
int g_nontemporal = -1;   // -1: streaming accesses only when the buffers cannot all sit in the Infinity Cache
int g_sched_variant = 0;  // 0 = pick the scheduler shape from the chunk count
int g_sched_uniform_fast = 1;
int g_copy_uniform_grid = 1;


// Per-launch timing: while a profiling region is open on the calling thread, every kernel is launched
// with its own start/stop events (hipExtLaunchKernelGGL), which bracket the kernel alone and not the
// gaps around it.  The events are read back when the region is closed, so the launches themselves
// stay asynchronous and back to back.
struct ProfRec { hipEvent_t e0, e1; int kid; };
thread_local std::vector<ProfRec>* g_prof_ring = nullptr;
thread_local size_t g_prof_n = 0;
thread_local bool g_prof_on = false;
thread_local int g_prof_kid = 0;   // which entry point is launching: 1 schedule, 2 stripe, 3 reassemble, 4 gather, 5 scatter, 6 copy

#define FL_LAUNCH(kernel, grid, block, shmem, stream, ...)                                              \
  do {                                                                                                  \
    if (g_prof_on && g_prof_n < g_prof_ring->size()) {                                                  \
      ProfRec& pr_ = (*g_prof_ring)[g_prof_n++];                                                        \
      pr_.kid = g_prof_kid;                                                                             \
      hipExtLaunchKernelGGL(kernel, grid, block, shmem, stream, pr_.e0, pr_.e1, 0, __VA_ARGS__);        \
    } else {                                                                                            \
      hipLaunchKernelGGL(kernel, grid, block, shmem, stream, __VA_ARGS__);                              \
    }                                                                                                   \
  } while (0)

int64_t env_i64(const char* name, int64_t dflt) {
  const char* v = getenv(name);
  if (!v || !*v) return dflt;
  char* end = nullptr;
  long long x = strtoll(v, &end, 0);
  return end && *end == 0 ? x : dflt;
}

}  // namespace

int fl_set_error(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

#define FL_HIP(call)                                                                         \
  do {                                                                                       \
    hipError_t e_ = (call);                                                                  \
    if (e_ != hipSuccess)                                                                    \
      return fl_set_error(e_ == hipErrorNoDevice ? FLH_E_NODEV : FLH_E_HIP, "%s failed: %s (%s:%d)", #call, \
                          hipGetErrorString(e_), __FILE__, __LINE__);                        \
  } while (0)

extern "C" {

const char* flh_last_error(void) { return g_err; }

int64_t flh_constant(int which) {
  switch (which) {
    case 0: return FLH_TILE_BYTES;
    case 1: return FLH_MAX_LANES;
    case 2: return FLH_UNIT_BYTES;
    case 3: return FLH_POOL_UNITS;
    case 4: return sizeof(flh_chunk_desc);
    case 5: return sizeof(flh_sched_state);
    case 6: return sizeof(flh_sched_hdr);
    case 7: return 1;
    case 8: return sizeof(flh_windows);
    case 9: return sizeof(flh_sched_params);
  }
  return -1;
}

int flh_init(int device) {
  int count = 0;
  hipError_t e = hipGetDeviceCount(&count);
  if (e != hipSuccess || count == 0)
    return fl_set_error(FLH_E_NODEV, "no HIP device: %s", e == hipSuccess ? "device count is 0" : hipGetErrorString(e));
  if (device < 0 || device >= count) return fl_set_error(FLH_E_ARG, "device %d out of range (%d devices)", device, count);
  FL_HIP(hipSetDevice(device));
  hipDeviceProp_t prop;
  FL_HIP(hipGetDeviceProperties(&prop, device));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return fl_set_error(FLH_E_NODEV, "device %d is %s; this library carries gfx950 code only", device, prop.gcnArchName);
  g_device = device;
  g_cus = prop.multiProcessorCount;
  g_grid_per_cu = (int)env_i64("NCCL_FUSELINK_GRID_PER_CU", g_grid_per_cu);
  g_nontemporal = (int)env_i64("NCCL_FUSELINK_NONTEMPORAL", g_nontemporal);
  if (g_grid_per_cu < 0) g_grid_per_cu = 0;
  return FLH_OK;
}

int flh_prof_begin(int capacity) {
  if (capacity < 1 || capacity > (1 << 20)) return fl_set_error(FLH_E_ARG, "capacity %d out of range", capacity);
  if (!g_prof_ring) g_prof_ring = new std::vector<ProfRec>();
  while (g_prof_ring->size() < (size_t)capacity) {
    ProfRec r;
    r.kid = 0;
    FL_HIP(hipEventCreate(&r.e0));
    FL_HIP(hipEventCreate(&r.e1));
    g_prof_ring->push_back(r);
  }
  g_prof_n = 0;
  g_prof_on = true;
  return FLH_OK;
}

int flh_prof_end(double* us_out, int* kernel_out, int max) {
  g_prof_on = false;
  if (!g_prof_ring) return fl_set_error(FLH_E_STATE, "no profiling region was opened on this thread");
  const size_t n = g_prof_n;
  for (size_t i = 0; i < n; ++i) {
    ProfRec& r = (*g_prof_ring)[i];
    FL_HIP(hipEventSynchronize(r.e1));
    float ms = 0.f;
    FL_HIP(hipEventElapsedTime(&ms, r.e0, r.e1));
    if ((int)i < max) {
      if (us_out) us_out[i] = (double)ms * 1e3;
      if (kernel_out) kernel_out[i] = r.kid;
    }
  }
  g_prof_n = 0;
  return (int)n;
}

int flh_tune(const char* key, int64_t value) {
  if (!key) return fl_set_error(FLH_E_ARG, "null key");
  if (!strcmp(key, "grid_per_cu")) { if (value < 0) return fl_set_error(FLH_E_ARG, "grid_per_cu < 0"); g_grid_per_cu = (int)value; return FLH_OK; }
  if (!strcmp(key, "stripe_dest_order")) { g_dest_order = value < 0 ? -1 : (value != 0); return FLH_OK; }
  if (!strcmp(key, "fused_fast")) { g_fused_fast = value != 0; return FLH_OK; }
  if (!strcmp(key, "nontemporal")) { g_nontemporal = value < 0 ? -1 : (value != 0); return FLH_OK; }
  if (!strcmp(key, "copy_uniform_grid")) { g_copy_uniform_grid = value != 0; return FLH_OK; }
  if (!strcmp(key, "sched_uniform_fast")) { g_sched_uniform_fast = value != 0; return FLH_OK; }
  if (!strcmp(key, "sched_variant")) { if (value < 0 || value > 4) return fl_set_error(FLH_E_ARG, "sched_variant not in 0..4"); g_sched_variant = (int)value; return FLH_OK; }
  return fl_set_error(FLH_E_ARG, "unknown tunable %s", key);
}

static int need_init() {
  if (g_device < 0) {
    int rc = flh_init((int)env_i64("NCCL_FUSELINK_DEVICE", 0));
    if (rc) return rc;
  }
  return FLH_OK;
}

int flh_schedule(const flh_sched_params* p, void* stream) {
  if (!p) return fl_set_error(FLH_E_ARG, "null params");
  if (p->n_lanes == 0 || p->n_lanes > FLH_MAX_LANES) return fl_set_error(FLH_E_ARG, "n_lanes %u not in 1..%d", p->n_lanes, FLH_MAX_LANES);
  if (p->n_rows == 0) return fl_set_error(FLH_E_ARG, "credit table missing");
  if (!p->d_credits && p->n_rows != 1) return fl_set_error(FLH_E_ARG, "inline credits carry exactly one row");
  if (p->quantum == 0) return fl_set_error(FLH_E_ARG, "quantum must be > 0");
  if (p->tile_bytes == 0 || p->tile_bytes % 128) return fl_set_error(FLH_E_ARG, "tile_bytes %u must be a positive multiple of 128", p->tile_bytes);
  if (!p->d_hdr || (p->n_chunks && !p->d_table)) return fl_set_error(FLH_E_ARG, "output pointers missing");
  if (!p->d_sizes) {
    if (p->n_chunks && p->chunk_bytes == 0) return fl_set_error(FLH_E_ARG, "chunk_bytes must be > 0 for the uniform split");
    const uint64_t need = p->chunk_bytes ? (p->total_bytes + p->chunk_bytes - 1) / p->chunk_bytes : 0;
    if (need != p->n_chunks) return fl_set_error(FLH_E_ARG, "n_chunks %u does not match ceil(%llu / %u) = %llu", p->n_chunks,
                                                (unsigned long long)p->total_bytes, p->chunk_bytes, (unsigned long long)need);
  }
  int rc = need_init();
  if (rc) return rc;
  g_prof_kid = 1;
  SchedArgs a;
  a.sizes = p->d_sizes;
  a.total_bytes = p->total_bytes;
  a.src_off = p->d_src_off;
  a.src_base = p->src_base;
  a.credits = p->d_credits;
  a.quantum = p->quantum;
  a.state = p->d_state;
  a.table = p->d_table;
  a.hdr = p->d_hdr;
  a.table_by_lane = p->d_table_by_lane;
  a.chunk_bytes = p->chunk_bytes;
  a.n = p->n_chunks;
  a.n_lanes = p->n_lanes;
  a.n_rows = p->n_rows;
  a.epoch_len = p->epoch_len;
  a.tile_bytes = p->tile_bytes;
  a.mode = p->mode;
  for (int l = 0; l < FLH_MAX_LANES; ++l) a.inline_credits[l] = p->inline_credits[l];
  a.quantum_shift = (p->quantum & (p->quantum - 1)) == 0 ? __builtin_ctzll(p->quantum) : -1;
  hipStream_t s = (hipStream_t)stream;
  a.tile_shift = (p->tile_bytes & (p->tile_bytes - 1)) == 0 ? __builtin_ctz(p->tile_bytes) : -1;
  const uint32_t n = p->n_chunks;
  const int variant = g_sched_variant;
  // ordinary message split with quantum-sized chunks: closed form, no scan
  if (g_sched_uniform_fast && variant == 0 && n > 0 && !p->d_sizes && !p->d_src_off && p->quantum == p->chunk_bytes &&
      p->n_rows <= (uint32_t)kRowCache) {
    const uint32_t grid = (n + kUniBlock - 1) / kUniBlock;
    FL_LAUNCH((fl_schedule_uniform_kernel<0>), dim3(grid), dim3(kUniBlock), 0, s, a);
    if (grid > 1 && p->d_state) FL_LAUNCH((fl_schedule_uniform_kernel<1>), dim3(1), dim3(kUniBlock), 0, s, a);
    FL_HIP(hipGetLastError());
    return FLH_OK;
  }
  if (p->d_table_by_lane && n > 0) return fl_set_error(FLH_E_ARG, "d_table_by_lane needs the uniform closed-form split (no d_sizes, no d_src_off, quantum == chunk_bytes, n_rows <= %d)", kRowCache);
  // one workgroup; more chunks per thread once the per-pass overhead stops dominating
  if ((variant == 0 && n <= kWave) || variant == 1) {
    FL_LAUNCH((fl_schedule_kernel<1, 1>), dim3(1), dim3(kWave), 0, s, a);
  } else if ((variant == 0 && n <= 8 * kWave) || variant == 2) {
    FL_LAUNCH((fl_schedule_kernel<4, 1>), dim3(1), dim3(4 * kWave), 0, s, a);
  } else if ((variant == 0 && n <= 32 * kWave) || variant == 3) {
    FL_LAUNCH((fl_schedule_kernel<8, 4>), dim3(1), dim3(8 * kWave), 0, s, a);
  } else {
    FL_LAUNCH((fl_schedule_kernel<8, 8>), dim3(1), dim3(8 * kWave), 0, s, a);
  }
  FL_HIP(hipGetLastError());
  return FLH_OK;
}

static int check_windows(const flh_windows* win) {
  if (!win) return fl_set_error(FLH_E_ARG, "null windows");
  if (win->n_lanes == 0 || win->n_lanes > FLH_MAX_LANES) return fl_set_error(FLH_E_ARG, "windows.n_lanes %u not in 1..%d", win->n_lanes, FLH_MAX_LANES);
  for (uint32_t l = 0; l < win->n_lanes; ++l)
    if (!win->base[l] && win->cap[l]) return fl_set_error(FLH_E_ARG, "window %u has capacity but no base", l);
  return FLH_OK;
}

// Non-temporal loads and stores pay off once the working set (the buffers a transfer touches) is well
// beyond the 256 MB Infinity Cache (measured: +3-5 % at 1 GiB messages) and cost throughput when a
// good part of it still fits (-8 % at 64 MiB, -20 % on the read-back side at 128 MiB).
static bool use_nt(uint64_t working_set_bytes) {
  if (g_nontemporal >= 0) return g_nontemporal != 0;
  return working_set_bytes > kCacheResidentBytes;
}

static uint32_t copy_grid(uint64_t max_tiles) {
  // one workgroup per tile lets the dispatcher overlap loads and stores of different tiles; the
  // kernels' stride loops only matter beyond the cap (grid_per_cu can lower it for experiments)
  uint64_t g = g_grid_per_cu > 0 ? (uint64_t)g_cus * (uint64_t)g_grid_per_cu : (1ull << 20);
  if (g > max_tiles) g = max_tiles;
  if (g < 1) g = 1;
  return (uint32_t)g;
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
  rc = need_init();
  if (rc) return rc;
  g_prof_kid = dir == 0 ? 2 : 3;
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
  const uint64_t max_tiles = h_hdr ? h_hdr->total_tiles : user_bytes / tile_bytes + n_chunks_max;
  if (max_tiles == 0) return FLH_OK;
  hipStream_t s = (hipStream_t)stream;
  const bool nt = use_nt(3 * user_bytes);  // user buffer + windows + the peer's buffer
  if (h_hdr && h_hdr->uniform_tiles && h_hdr->n_chunks <= 65535 && h_hdr->n_chunks <= n_chunks_max && g_copy_uniform_grid) {
    const dim3 grid(h_hdr->uniform_tiles, h_hdr->n_chunks);
    if (dir == 0) {
      if (nt) FL_LAUNCH((fl_copy_uniform<0, true>), grid, dim3(kCopyBlock), 0, s, a);
      else FL_LAUNCH((fl_copy_uniform<0, false>), grid, dim3(kCopyBlock), 0, s, a);
    } else {
      if (nt) FL_LAUNCH((fl_copy_uniform<1, true>), grid, dim3(kCopyBlock), 0, s, a);
      else FL_LAUNCH((fl_copy_uniform<1, false>), grid, dim3(kCopyBlock), 0, s, a);
    }
    FL_HIP(hipGetLastError());
    return FLH_OK;
  }
  const uint32_t grid = copy_grid(max_tiles);
  if (dir == 0) {
    if (nt) FL_LAUNCH((fl_copy_tiles<0, true>), dim3(grid), dim3(kCopyBlock), 0, s, a);
    else FL_LAUNCH((fl_copy_tiles<0, false>), dim3(grid), dim3(kCopyBlock), 0, s, a);
  } else {
    if (nt) FL_LAUNCH((fl_copy_tiles<1, true>), dim3(grid), dim3(kCopyBlock), 0, s, a);
    else FL_LAUNCH((fl_copy_tiles<1, false>), dim3(grid), dim3(kCopyBlock), 0, s, a);
  }
  FL_HIP(hipGetLastError());
  return FLH_OK;
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
                      flh_sched_hdr* d_hdr, int32_t* d_status) {
  int rc = check_windows(win);
  if (rc) return rc;
  if (!u || !d_status) return fl_set_error(FLH_E_ARG, "parameters and d_status are required");
  if (u->n_lanes == 0 || u->n_lanes > FLH_MAX_LANES || u->n_lanes != win->n_lanes) return fl_set_error(FLH_E_ARG, "n_lanes %u does not match the windows' %u", u->n_lanes, win->n_lanes);
  if (u->chunk_bytes == 0) return fl_set_error(FLH_E_ARG, "chunk_bytes must be > 0");
  if (u->tile_bytes == 0 || u->tile_bytes % 128) return fl_set_error(FLH_E_ARG, "tile_bytes %u must be a positive multiple of 128", u->tile_bytes);
  if (u->total_bytes == 0) return 1;
  const uint64_t n = (u->total_bytes + u->chunk_bytes - 1) / u->chunk_bytes;
  if (n > 65535) return fl_set_error(FLH_E_ARG, "%llu chunks exceed the 65535 one launch can name; split the message", (unsigned long long)n);
  rc = need_init();
  if (rc) return rc;
  g_prof_kid = dir == 0 ? 2 : 3;
  a.user = nullptr;
  a.user_bytes = 0;
  a.win = *win;
  a.table = dir == 0 ? d_table : nullptr;
  a.hdr = dir == 0 ? d_hdr : nullptr;
  a.status = d_status;
  a.total_bytes = u->total_bytes;
  a.src_base = u->src_base;
  a.quanta_before = u->epoch_bytes / u->chunk_bytes;
  a.chunk_bytes = u->chunk_bytes;
  a.n_chunks = (uint32_t)n;
  a.n_lanes = u->n_lanes;
  a.tile_bytes = u->tile_bytes;
  a.tiles_per_chunk = (u->chunk_bytes + u->tile_bytes - 1) / u->tile_bytes;
  // once the message no longer fits the Infinity Cache, write every window front to back
  a.dest_order = dir == 0 && (g_dest_order < 0 ? 3 * u->total_bytes > kCacheResidentBytes : g_dest_order != 0);
  for (int l = 0; l < FLH_MAX_LANES; ++l) a.credits[l] = (uint32_t)l < u->n_lanes ? u->credits[l] : 0;
  {
    // the row as the kernel sees it (equal credits stand in for an all-zero row), then the host-side constants
    uint64_t pfx[FLH_MAX_LANES], W = 0;
    for (uint32_t l = 0; l < u->n_lanes; ++l) { W += u->credits[l]; pfx[l] = W; }
    if (W == 0) { for (uint32_t l = 0; l < u->n_lanes; ++l) pfx[l] = l + 1; W = u->n_lanes; }
    a.fast = W >= 2 && W <= 0xffffffffull && a.quanta_before + n <= 0xffffffffull && g_fused_fast;
    a.magic = a.fast ? ~0ull / W + 1 : 0;
    for (int l = 0; l < FLH_MAX_LANES; ++l) a.cnt0[l] = 0;
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
static int launch_fused_args(int dir, const Args& a, bool nt, void* stream) {
  const dim3 grid(a.tiles_per_chunk, a.n_chunks);
  hipStream_t s = (hipStream_t)stream;
  if (dir == 0) {
    if (nt) FL_LAUNCH((fl_copy_uniform_fused<0, true, Args>), grid, dim3(kCopyBlock), 0, s, a);
    else FL_LAUNCH((fl_copy_uniform_fused<0, false, Args>), grid, dim3(kCopyBlock), 0, s, a);
  } else {
    if (nt) FL_LAUNCH((fl_copy_uniform_fused<1, true, Args>), grid, dim3(kCopyBlock), 0, s, a);
    else FL_LAUNCH((fl_copy_uniform_fused<1, false, Args>), grid, dim3(kCopyBlock), 0, s, a);
  }
  FL_HIP(hipGetLastError());
  return FLH_OK;
}
}  // extern "C++"

static int launch_fused(int dir, void* user, uint64_t user_bytes, const flh_windows* win, const flh_uniform_params* u,
                        flh_chunk_desc* d_table, flh_sched_hdr* d_hdr, int32_t* d_status, void* stream) {
  FusedArgs a;
  const int rc = fill_fused(a, dir, win, u, d_table, d_hdr, d_status);
  if (rc) return rc < 0 ? rc : FLH_OK;
  if (!user) return fl_set_error(FLH_E_ARG, "user buffer missing");
  a.user = (uint8_t*)user;
  a.user_bytes = user_bytes;
  return launch_fused_args(dir, a, use_nt(3 * user_bytes), stream);
}

static int launch_batch(int dir, const flh_batch_params* b, const flh_windows* win, flh_chunk_desc* d_table, flh_sched_hdr* d_hdr,
                        int32_t* d_status, void* stream) {
  if (!b) return fl_set_error(FLH_E_ARG, "null batch");
  if (b->n_req == 0 || b->n_req > FLH_BATCH_MAX) return fl_set_error(FLH_E_ARG, "n_req %u not in 1..%d", b->n_req, FLH_BATCH_MAX);
  FusedBatchArgs a;
  const int rc = fill_fused(a, dir, win, &b->u, d_table, d_hdr, d_status);
  if (rc) return rc < 0 ? rc : FLH_OK;
  a.dest_order = 0;
  a.src_base = 0;
  a.n_req = b->n_req;
  uint64_t sum = 0;
  for (uint32_t q = 0; q < FLH_BATCH_MAX; ++q) {
    a.first[q] = 0;
    a.req_user[q] = nullptr;
    a.req_bytes[q] = 0;
    if (q >= b->n_req) continue;
    void* p = dir == 0 ? (void*)b->d_src[q] : b->d_dst[q];
    if (!p || b->bytes[q] == 0) return fl_set_error(FLH_E_ARG, "request %u of the batch has no buffer or no bytes", q);
    if (q + 1 < b->n_req && b->bytes[q] % b->u.chunk_bytes) return fl_set_error(FLH_E_ARG, "request %u of the batch is not a whole number of chunks", q);
    a.first[q] = (uint32_t)(sum / b->u.chunk_bytes);
    a.req_user[q] = (uint8_t*)p;
    a.req_bytes[q] = b->bytes[q];
    sum += b->bytes[q];
  }
  if (sum != b->u.total_bytes) return fl_set_error(FLH_E_ARG, "the requests hold %llu bytes, the parameters say %llu", (unsigned long long)sum, (unsigned long long)b->u.total_bytes);
  return launch_fused_args(dir, a, use_nt(3 * sum), stream);
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
  rc = need_init();
  if (rc) return rc;
  g_prof_kid = dir == 0 ? 4 : 5;
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
  const uint64_t total = (uint64_t)n_chunks * pages_per_chunk * a.subs_per_page;
  const uint32_t grid = copy_grid(total);
  hipStream_t s = (hipStream_t)stream;
  const bool nt = use_nt(3ull * n_chunks * pages_per_chunk * page_bytes);
#define FL_LAUNCH_PAGES(D, LD, N) FL_LAUNCH((fl_page_tiles<D, LD, N>), dim3(grid), dim3(kCopyBlock), 0, s, a)
  if (dir == 0) {
    if (use_lds) { if (nt) FL_LAUNCH_PAGES(0, true, true); else FL_LAUNCH_PAGES(0, true, false); }
    else { if (nt) FL_LAUNCH_PAGES(0, false, true); else FL_LAUNCH_PAGES(0, false, false); }
  } else {
    if (use_lds) { if (nt) FL_LAUNCH_PAGES(1, true, true); else FL_LAUNCH_PAGES(1, true, false); }
    else { if (nt) FL_LAUNCH_PAGES(1, false, true); else FL_LAUNCH_PAGES(1, false, false); }
  }
#undef FL_LAUNCH_PAGES
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

int flh_copy(void* d_dst, const void* d_src, uint64_t bytes, void* stream) {
  if (bytes == 0) return FLH_OK;
  if (!d_dst || !d_src) return fl_set_error(FLH_E_ARG, "null pointer");
  int rc = need_init();
  if (rc) return rc;
  g_prof_kid = 6;
  const uint32_t tile = FLH_TILE_BYTES;
  const uint32_t grid = copy_grid((bytes + tile - 1) / tile);
  hipStream_t s = (hipStream_t)stream;
  if (use_nt(2 * bytes)) FL_LAUNCH(fl_plain_copy<true>, dim3(grid), dim3(kCopyBlock), 0, s, (uint8_t*)d_dst, (const uint8_t*)d_src, bytes, tile);
  else FL_LAUNCH(fl_plain_copy<false>, dim3(grid), dim3(kCopyBlock), 0, s, (uint8_t*)d_dst, (const uint8_t*)d_src, bytes, tile);
  FL_HIP(hipGetLastError());
  return FLH_OK;
}

int flh_qp_split(int size, int nqps, int* off, int* len) {
  if (nqps < 1 || size < 0 || !off || !len) return fl_set_error(FLH_E_ARG, "bad qp split arguments");
  // stride = ceil(ceil(size / nqps) / 128) * 128; a piece past the end is an empty work request.
  // 64-bit inside: the reference's `int` expression overflows for sizes within 127 bytes of INT_MAX.
  const int64_t per = ((int64_t)size + nqps - 1) / nqps;
  const int64_t stride = (per + 127) / 128 * 128;
  int64_t o = 0;
  for (int q = 0; q < nqps; ++q, o += stride) {
    int64_t l = (int64_t)size - o;
    if (l > stride) l = stride;
    off[q] = o > 0x7fffffff ? 0x7fffffff : (int)o;
    len[q] = l > 0 ? (int)l : 0;
  }
  return stride > 0x7fffff80 ? 0x7fffff80 : (int)stride;
}

}  // extern "C"
