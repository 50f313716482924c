// fl_sched.hip -- the chunk -> (lane, window offset) scheduler kernels and flh_schedule:
//   * fl_schedule_kernel         : any chunk sizes; one workgroup, wavefront prefix scans (DPP)
//   * fl_schedule_uniform_kernel : uniform split with quantum-sized chunks; closed form, any number of workgroups
// All cross-lane traffic is DPP row shifts and row broadcasts; LDS only passes per-wavefront totals between the
// wavefronts of the one workgroup and caches the credit rows.
#include <atomic>
#include <cstring>

#include "fl_device.h"
#include "fl_launch.h"

namespace {

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
  struct SegHeader* seg;                   // caller's workspace when several workgroups share the scan, else null
  uint32_t wave_chunks;                    // uniform kernel: window offsets restart every so many chunks (0: never)
};

// Scan scheduler over several workgroups: the chunk list is cut into segments of kSegChunks, one workgroup each.
// What a segment needs from the ones before it -- bytes of its epoch so far, bytes and tiles of the call so far --
// depends on the sizes alone and is summed first (fl_sched_seg_totals); the segments are then scheduled side by
// side with window offsets counted from zero (fl_schedule_kernel, which leaves its per-lane totals here), and a
// last launch adds every lane's bytes of the earlier segments to the rows and writes header and state
// (fl_sched_seg_finish).  Three launches and no waiting between workgroups.
constexpr uint32_t kSegChunks = 1024;      // = one pass of fl_schedule_kernel<8, 2>
struct SegPartial {
  uint64_t bytes;          // of the whole segment
  uint64_t tail;           // from the segment's last epoch head on (the whole segment if it has none)
  uint32_t tiles;
  uint32_t has_head;
  uint64_t lane_bytes[FLH_MAX_LANES];
  uint32_t lane_chunks[FLH_MAX_LANES];
  uint32_t flags;
  uint32_t pad;
};
struct SegHeader {         // the carried state as it was when the call began
  uint64_t lane_off[FLH_MAX_LANES];
  uint64_t epoch_bytes;
  uint64_t chunk_index;
  SegPartial part[1];      // one per segment follows
};
__host__ __device__ inline uint32_t seg_count(uint32_t n) { return (n + kSegChunks - 1) / kSegChunks; }

// The workspace that flh_schedule_static brings along for callers that cannot allocate one: one copy per GPU, held until
// the process ends, sized for FLH_SCHED_STATIC_MAX_CHUNKS chunks.  In host code `scratch` is only a handle for
// hipGetSymbolAddress; the address the kernels get is the per-device one kept in g_scratch_ptr.
constexpr uint64_t kScratchBytes = sizeof(SegHeader) + (uint64_t)(FLH_SCHED_STATIC_MAX_CHUNKS / kSegChunks) * sizeof(SegPartial);
static_assert(FLH_SCHED_STATIC_MAX_CHUNKS % kSegChunks == 0, "the limit is a whole number of segments");
static_assert(kScratchBytes <= 256u * 1024u, "the static workspace is meant to stay modest");
static __device__ __align__(256) unsigned char scratch[kScratchBytes];
constexpr int kScratchDevices = 64;
std::atomic<void*> g_scratch_ptr[kScratchDevices];



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

// The same result for threads that own several chunks (K >= 4), with work per thread of K + L instead of K * L:
// every thread keeps one running byte count per lane in its own column of `acc` (LDS, [lane][thread], so the
// columns never collide and a wavefront's accesses fall on distinct banks), hands each chunk the count found
// there, then the per-lane scans run over the threads' column totals and their exclusive results are added back.
// 32-bit sums only: the caller takes the other routine when a pass moves 4 GiB or more.
template <int K, int BT>
__device__ __forceinline__ void lane_pass_columns(const uint32_t (&s)[K], const uint32_t (&ln)[K], uint32_t L, int tid, int lane,
                                                  uint32_t* acc, uint64_t* w_lane_row, uint64_t (&off)[K]) {
  constexpr int G = 4;
#pragma unroll 1
  for (uint32_t l = 0; l < L; ++l) acc[l * BT + tid] = 0;
#pragma unroll
  for (int k = 0; k < K; ++k) {
    if (ln[k] < L) {   // chunks past the end carry the lane "none"
      uint32_t* p = &acc[ln[k] * BT + tid];
      const uint32_t o = *p;
      off[k] = o;
      *p = o + s[k];
    }
  }
  uint64_t my_total = 0;
#pragma unroll 1
  for (uint32_t l0 = 0; l0 < L; l0 += G) {
    uint32_t v[G], inc[G];
#pragma unroll
    for (int g = 0; g < G; ++g) v[g] = l0 + g < L ? acc[(l0 + g) * BT + tid] : 0;
#pragma unroll
    for (int g = 0; g < G; ++g) inc[g] = wave_incl_sum_u32(v[g], lane);
#pragma unroll
    for (int g = 0; g < G; ++g) {
      if (l0 + g < L) acc[(l0 + g) * BT + tid] = inc[g] - v[g];
      const uint32_t tot = bcast_lane_u32(inc[g], kWave - 1);
      if ((uint32_t)lane == l0 + g) my_total = tot;
    }
  }
#pragma unroll
  for (int k = 0; k < K; ++k) {
    if (ln[k] < L) off[k] += acc[ln[k] * BT + tid];
  }
  if ((uint32_t)lane < L) w_lane_row[lane] = my_total;
}

// One workgroup of NW wavefronts walks the chunk list in passes of NW*64*K chunks; thread t owns K
// consecutive chunks of a pass.  Per pass: thread-local sums, three wavefront scans (epoch-segmented
// bytes, bytes, tiles), the lane of each chunk from its quantum slot, one wavefront scan per lane
// for the window offsets.  LDS only carries per-wavefront totals and the running lane offsets.
template <int NW, int K, bool SEG = false>
__global__ __launch_bounds__(NW * kWave) void fl_schedule_kernel(SchedArgs a) {
  warm_kernel_args(a);
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
  __shared__ uint32_t acc[K >= 4 ? FLH_MAX_LANES * BT : 1];   // per-thread, per-lane running byte counts (lane_pass_columns)

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
  // this workgroup's part of the chunk list: all of it, or one segment
  uint32_t n_loc = a.n, i_base = 0;
  const uint32_t* sizes_p = a.sizes;
  const uint64_t* srcoff_p = a.src_off;
  flh_chunk_desc* table_p = a.table;
  if constexpr (SEG) {
    const uint32_t g = blockIdx.x;
    i_base = g * kSegChunks;
    n_loc = a.n - i_base < kSegChunks ? a.n - i_base : kSegChunks;
    if (sizes_p) sizes_p += i_base;
    if (srcoff_p) srcoff_p += i_base;
    table_p += i_base;
    off_in = 0;   // window offsets are counted from zero here; the finishing launch adds what lies before
    k0 += i_base;
  }
  uint32_t s_next[K];
#pragma unroll
  for (int k = 0; k < K; ++k) {
    const uint32_t i = (uint32_t)tid * K + k;
    s_next[k] = (sizes_p && i < n_loc) ? sizes_p[i] : 0;
  }
  if constexpr (SEG) {
    // What the earlier segments hand over: their bytes and tiles, and the bytes since the last epoch head among
    // them.  One wavefront reads their partials sixty-four at a time (one round trip for up to 65 536 chunks).
    const uint32_t g = blockIdx.x;
    __shared__ uint64_t c_run, c_p;
    __shared__ uint32_t c_tiles;
    if (wave == 0) {
      uint64_t run = 0, after = 0;
      uint32_t tiles = 0;
      bool seen_head = false;
      for (uint32_t base = 0; base < g; base += kWave) {
        const uint32_t q = base + lane;
        uint64_t b = 0, tl = 0;
        uint32_t t = 0, hd = 0;
        if (q < g) {
          const SegPartial& pq = a.seg->part[q];
          b = pq.bytes;
          tl = pq.tail;
          t = pq.tiles;
          hd = pq.has_head;
        }
        const uint64_t heads = __builtin_amdgcn_ballot_w64(hd != 0);
        run += bcast_lane_u64(wave_incl_sum_u64(b, lane), kWave - 1);
        tiles += bcast_lane_u32(wave_incl_sum_u32(t, lane), kWave - 1);
        if (heads) {
          const int hb = 63 - __builtin_clzll(heads);
          const uint64_t above = bcast_lane_u64(wave_incl_sum_u64(lane > hb ? b : 0, lane), kWave - 1);
          after = bcast_lane_u64(tl, hb) + above;
          seen_head = true;
        } else {
          after += bcast_lane_u64(wave_incl_sum_u64(b, lane), kWave - 1);
        }
      }
      if (lane == 0) {
        c_run = run;
        c_tiles = tiles;
        c_p = seen_head ? after : p_carry + after;
      }
    }
    __syncthreads();
    p_carry = c_p;
    run_carry = c_run;
    tiles_carry = c_tiles;
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
  for (uint32_t pass = 0; pass < n_loc; pass += BT * K) {
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
      if (i < n_loc) {
        if (sizes_p) {
          sz = s_next[k];
        } else {
          const uint64_t o = (uint64_t)(i_base + i) * a.chunk_bytes;
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
    if (sizes_p) {  // next pass's sizes travel while this pass computes
#pragma unroll
      for (int k = 0; k < K; ++k) {
        const uint64_t i = (uint64_t)i0 + (uint64_t)BT * K + k;
        s_next[k] = i < n_loc ? sizes_p[i] : 0;
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
      if (i < n_loc) {
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
    if constexpr (K >= 4) {
      if ((tot_run >> 32) == 0) lane_pass_columns<K, BT>(s, ln, L, tid, lane, acc, w_lane[wave], off);
      else lane_pass<uint64_t, K>(s, ln, L, lane, w_lane[wave], off);
    } else {
      if ((tot_run >> 32) == 0) lane_pass<uint32_t, K>(s, ln, L, lane, w_lane[wave], off);
      else lane_pass<uint64_t, K>(s, ln, L, lane, w_lane[wave], off);
    }
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
      if (i < n_loc) {
        flh_chunk_desc d;
        d.src_off = srcoff_p ? srcoff_p[i] : a.src_base + run_i;
        d.win_off = (a.mode & FLH_SCHED_MIRROR) ? d.src_off : w_lane[wave][ln[k]] + off[k];
        d.len = s[k];
        d.lane = ln[k];
        d.tile_base = tiles_i;
        d.epoch = ep[k];
        table_p[i] = d;
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
  if constexpr (SEG) {   // one segment of several: its per-lane totals go to the workspace, header and state wait for the last launch
    SegPartial& me = a.seg->part[blockIdx.x];
    if (tid < FLH_MAX_LANES) {
      me.lane_bytes[tid] = lane_off[tid];
      me.lane_chunks[tid] = cnt_lane[tid];
    }
    if (tid == 0) me.flags = sh_flags;
    return;
  }
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
// scan scheduler over several workgroups: first and last launch
// ------------------------------------------------------------------------------------------------
constexpr int kSegBlock = 256;

__device__ __forceinline__ uint32_t seg_chunk_size(const SchedArgs& a, uint32_t i) {
  if (a.sizes) return a.sizes[i];
  const uint64_t o = (uint64_t)i * a.chunk_bytes;
  const uint64_t rem = o < a.total_bytes ? a.total_bytes - o : 0;
  return (uint32_t)(rem < a.chunk_bytes ? rem : a.chunk_bytes);
}

// Per segment: bytes, tiles, and the bytes from its last epoch head on.  Epoch heads sit at fixed chunk indices
// (multiples of epoch_len counted from the carried chunk index), so the last one inside a segment is a division.
__global__ __launch_bounds__(kSegBlock) void fl_sched_seg_totals(SchedArgs a) {
  warm_kernel_args(a);
  const uint32_t g = blockIdx.x, tid = threadIdx.x;
  const uint32_t lo = g * kSegChunks;
  const uint32_t hi = a.n - lo < kSegChunks ? a.n : lo + kSegChunks;
  const uint64_t k0 = a.state ? a.state->chunk_index : 0;
  uint32_t has_head = 0, head_i = lo;
  if (a.epoch_len) {
    const uint64_t last = div_u64(k0 + hi - 1, a.epoch_len) * a.epoch_len;   // global index of the last head at or below hi - 1
    if (last >= k0 + lo) { has_head = 1; head_i = (uint32_t)(last - k0); }
  }
  constexpr int kWaves = kSegBlock / kWave;
  __shared__ uint64_t sh_bytes[kWaves], sh_tail[kWaves];
  __shared__ uint32_t sh_tiles[kWaves];
  uint64_t b = 0, tl = 0;
  uint32_t t = 0;
  for (uint32_t i = lo + tid; i < hi; i += kSegBlock) {
    const uint32_t sz = seg_chunk_size(a, i);
    b += sz;
    if (i >= head_i) tl += sz;
    t += a.tile_shift >= 0 ? (sz + a.tile_bytes - 1) >> a.tile_shift : (sz + a.tile_bytes - 1) / a.tile_bytes;
  }
  const int lane = tid & (kWave - 1);
  b = wave_incl_sum_u64(b, lane);
  tl = wave_incl_sum_u64(tl, lane);
  t = wave_incl_sum_u32(t, lane);
  if (lane == kWave - 1) { sh_bytes[tid / kWave] = b; sh_tail[tid / kWave] = tl; sh_tiles[tid / kWave] = t; }
  __syncthreads();
  if (tid == 0) {
    SegPartial& me = a.seg->part[g];
    uint64_t sb = 0, st = 0;
    uint32_t sn = 0;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) { sb += sh_bytes[w]; st += sh_tail[w]; sn += sh_tiles[w]; }
    me.bytes = sb;
    me.tail = st;
    me.tiles = sn;
    me.has_head = has_head;
  }
  if (g == 0) {   // the state as the call found it, for the launches that follow (the last of them overwrites the state)
    if (tid < FLH_MAX_LANES) a.seg->lane_off[tid] = (a.state && !(a.mode & FLH_SCHED_RESET_OFFSETS)) ? a.state->lane_off[tid] : 0;
    if (tid == 0) {
      a.seg->epoch_bytes = (a.state && !(a.mode & FLH_SCHED_NEW_EPOCH)) ? a.state->epoch_bytes : 0;
      a.seg->chunk_index = k0;
    }
  }
}

// Window offsets of a segment's rows start where the earlier segments left each lane; the workgroup of the first
// segment also sums everything up into header and state.
__global__ __launch_bounds__(kSegBlock) void fl_sched_seg_finish(SchedArgs a) {
  warm_kernel_args(a);
  const uint32_t g = blockIdx.x, tid = threadIdx.x, G = gridDim.x;
  const uint32_t lo = g * kSegChunks;
  const uint32_t hi = a.n - lo < kSegChunks ? a.n : lo + kSegChunks;
  // every lane's bytes in the earlier segments: thread (q, l) sums the segments q, q + 16, ... for lane l
  constexpr int kQ = kSegBlock / FLH_MAX_LANES;
  __shared__ uint64_t part_sum[kQ][FLH_MAX_LANES];
  __shared__ uint64_t base[FLH_MAX_LANES];
  {
    const uint32_t q = tid / FLH_MAX_LANES, l = tid % FLH_MAX_LANES;
    uint64_t v = 0;
    for (uint32_t s = q; s < g; s += kQ) v += a.seg->part[s].lane_bytes[l];
    part_sum[q][l] = v;
  }
  __syncthreads();
  if (tid < FLH_MAX_LANES) {
    uint64_t v = a.seg->lane_off[tid];
#pragma unroll
    for (int q = 0; q < kQ; ++q) v += part_sum[q][tid];
    base[tid] = v;
  }
  __syncthreads();
  if (!(a.mode & FLH_SCHED_MIRROR)) {
    for (uint32_t i = lo + tid; i < hi; i += kSegBlock) {
      const uint32_t ln = a.table[i].lane;
      a.table[i].win_off += base[ln < FLH_MAX_LANES ? ln : 0];
    }
  }
  if (g != 0) return;   // the first segment's workgroup had nothing to sum for its own rows: it sums up for all
  // ---- header and state, from every segment's partials ----------------------------------------------------
  __shared__ unsigned long long t_bytes, t_after, t_lane[FLH_MAX_LANES];
  __shared__ uint32_t t_tiles, t_flags, t_cnt[FLH_MAX_LANES];
  __shared__ int t_head;
  if (tid < FLH_MAX_LANES) { t_lane[tid] = 0; t_cnt[tid] = 0; }
  if (tid == 0) { t_bytes = 0; t_after = 0; t_tiles = 0; t_flags = 0; t_head = -1; }
  __syncthreads();
  {
    const uint32_t q = tid / FLH_MAX_LANES, l = tid % FLH_MAX_LANES;
    unsigned long long lb = 0, by = 0;
    uint32_t lc = 0, ti = 0, fl = 0;
    int hd = -1;
    for (uint32_t s = q; s < G; s += kQ) {
      const SegPartial& p = a.seg->part[s];
      lb += p.lane_bytes[l];
      lc += p.lane_chunks[l];
      if (l == 0) {
        by += p.bytes;
        ti += p.tiles;
        fl |= p.flags;
        if (p.has_head) hd = (int)s;
      }
    }
    if (lb) atomicAdd(&t_lane[l], lb);     // sixteen adds per lane at most
    if (lc) atomicAdd(&t_cnt[l], lc);
    if (l == 0) {
      if (by) atomicAdd(&t_bytes, by);
      if (ti) atomicAdd(&t_tiles, ti);
      if (fl) atomicOr(&t_flags, fl);
      if (hd >= 0) atomicMax(&t_head, hd);
    }
  }
  __syncthreads();
  const int h = t_head;
  {
    unsigned long long af = 0;
    for (uint32_t q = (uint32_t)(h + 1) + tid; q < G; q += kSegBlock) af += a.seg->part[q].bytes;
    if (af) atomicAdd(&t_after, af);
  }
  __syncthreads();
  if (tid < FLH_MAX_LANES) {
    a.hdr->lane_bytes[tid] = t_lane[tid];
    a.hdr->lane_chunks[tid] = t_cnt[tid];
    if (a.state) a.state->lane_off[tid] = a.seg->lane_off[tid] + t_lane[tid];
  }
  if (tid == 0) {
    a.hdr->total_bytes = t_bytes;
    a.hdr->total_tiles = t_tiles;
    a.hdr->n_chunks = a.n;
    a.hdr->flags = t_flags;
    a.hdr->uniform_tiles = (!a.sizes && a.n) ? (a.chunk_bytes + a.tile_bytes - 1) / a.tile_bytes : 0;
    if (a.state) {
      a.state->epoch_bytes = (h >= 0 ? a.seg->part[h].tail : a.seg->epoch_bytes) + t_after;
      a.state->chunk_index = a.seg->chunk_index + a.n;
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
  warm_kernel_args(a);
  __shared__ UniTables t;
  const int tid = threadIdx.x;
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
      uint64_t before = uni_before(t, c, i, 0xffffffffu, &ln, &ep);
      bool from_zero = !keep_off;
      if (a.wave_chunks) {   // the windows are reused wave by wave: count from the wave's first chunk, on an empty window
        const uint32_t w0 = i - i % a.wave_chunks;
        if (w0) { before -= uni_before(t, c, w0, ln, nullptr, nullptr); from_zero = true; }
      }
      const uint64_t o = (uint64_t)i * c.C;
      const uint64_t rem = a.total_bytes - o;
      flh_chunk_desc d;
      d.src_off = a.src_base + o;
      d.win_off = (a.mode & FLH_SCHED_MIRROR) ? d.src_off : (from_zero ? 0 : a.state->lane_off[ln]) + before * c.C;
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

}  // namespace

// ------------------------------------------------------------------------------------------------
// table -> per-tile descriptors
// ------------------------------------------------------------------------------------------------
// Eight lanes per row, striding over the row's tiles: a short row costs one store, a row of a thousand tiles 128 per
// lane.  Runs behind the scheduler kernel on the same stream and reads what that one wrote.
constexpr int kExpandBlock = 256;
constexpr int kExpandLanes = 8;
__global__ __launch_bounds__(kExpandBlock) void fl_expand_tiles(const flh_chunk_desc* __restrict__ table, const flh_sched_hdr* __restrict__ hdr,
                                                                uint32_t n_max, uint32_t tile_bytes, flh_tile_desc* __restrict__ out, uint32_t cap) {
  uint32_t n = hdr->n_chunks;
  if (n > n_max) n = n_max;
  const uint32_t lane = threadIdx.x & (kExpandLanes - 1);
  const uint32_t groups = gridDim.x * (kExpandBlock / kExpandLanes);
  for (uint32_t row = blockIdx.x * (kExpandBlock / kExpandLanes) + threadIdx.x / kExpandLanes; row < n; row += groups) {
    const flh_chunk_desc d = table[row];
    const uint32_t nt = (uint32_t)(((uint64_t)d.len + tile_bytes - 1) / tile_bytes);
    for (uint32_t j = lane; j < nt; j += kExpandLanes) {
      const uint32_t t = d.tile_base + j;
      if (t >= cap) break;
      const uint64_t off = (uint64_t)j * tile_bytes;
      flh_tile_desc o;
      o.src_off = d.src_off + off;
      o.win_off = d.win_off + off;
      o.len = (uint32_t)((d.len - off) < tile_bytes ? (d.len - off) : tile_bytes);
      o.lane = d.lane;
      o.row = row;
      o.pad = 0;
      out[t] = o;
    }
  }
}

extern "C" {

uint64_t flh_schedule_workspace_bytes(uint32_t n_chunks) {
  return sizeof(SegHeader) + (uint64_t)seg_count(n_chunks) * sizeof(SegPartial);
}

static int expand_tiles(const flh_sched_params* p, hipStream_t s) {
  if (!p->d_tiles || p->n_chunks == 0) return FLH_OK;
  const uint32_t per_block = kExpandBlock / kExpandLanes;
  uint32_t grid = (p->n_chunks + per_block - 1) / per_block;
  if (grid > 8192) grid = 8192;
  FL_LAUNCH(fl_expand_tiles, dim3(grid), dim3(kExpandBlock), 0, s, (const flh_chunk_desc*)p->d_table, (const flh_sched_hdr*)p->d_hdr, p->n_chunks,
            p->tile_bytes, p->d_tiles, p->tiles_cap);
  FL_HIP(hipGetLastError());
  return FLH_OK;
}

// flh_schedule with the workspace named apart from the parameters: the caller's (flh_schedule) or the library's own
// per-device array (flh_schedule_static).
static int schedule_with(const flh_sched_params* p, void* stream, void* d_workspace, uint64_t workspace_bytes) {
  if (!p) return fl_set_error(FLH_E_ARG, "null params");
  if (p->n_lanes == 0 || p->n_lanes > FLH_MAX_LANES) return fl_set_error(FLH_E_ARG, "n_lanes %u not in 1..%d", p->n_lanes, FLH_MAX_LANES);
  if (p->n_rows == 0) return fl_set_error(FLH_E_ARG, "credit table missing");
  if (!p->d_credits && p->n_rows != 1) return fl_set_error(FLH_E_ARG, "inline credits carry exactly one row");
  if (p->quantum == 0) return fl_set_error(FLH_E_ARG, "quantum must be > 0");
  if (p->tile_bytes == 0 || p->tile_bytes % 128) return fl_set_error(FLH_E_ARG, "tile_bytes %u must be a positive multiple of 128", p->tile_bytes);
  if (!p->d_hdr || (p->n_chunks && !p->d_table)) return fl_set_error(FLH_E_ARG, "output pointers missing");
  if (p->d_tiles && p->tiles_cap == 0) return fl_set_error(FLH_E_ARG, "d_tiles without tiles_cap");
  if (p->wave_chunks && (p->d_sizes || p->d_src_off || p->quantum != p->chunk_bytes || p->n_rows > (uint32_t)kRowCache || p->d_table_by_lane))
    return fl_set_error(FLH_E_ARG, "wave_chunks needs the uniform closed-form split (no d_sizes, no d_src_off, quantum == chunk_bytes, n_rows <= %d) and no d_table_by_lane", kRowCache);
  if (!p->d_sizes) {
    if (p->n_chunks && p->chunk_bytes == 0) return fl_set_error(FLH_E_ARG, "chunk_bytes must be > 0 for the uniform split");
    const uint64_t need = p->chunk_bytes ? (p->total_bytes + p->chunk_bytes - 1) / p->chunk_bytes : 0;
    if (need != p->n_chunks) return fl_set_error(FLH_E_ARG, "n_chunks %u does not match ceil(%llu / %u) = %llu", p->n_chunks,
                                                (unsigned long long)p->total_bytes, p->chunk_bytes, (unsigned long long)need);
  }
  int rc = fl_need_init();
  if (rc) return rc;
  fl_prof().kid = 1;
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
  a.seg = nullptr;
  a.wave_chunks = p->wave_chunks;
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
    return expand_tiles(p, s);
  }
  if (p->wave_chunks && n > 0) return fl_set_error(FLH_E_ARG, "wave_chunks: the closed-form scheduler is switched off by a tunable");
  // a long list with a workspace: one workgroup per kSegChunks chunks, three launches
  if (d_workspace && variant == 0 && n >= (uint32_t)g_sched_seg_min && p->n_rows <= (uint32_t)kRowCache && !p->d_table_by_lane) {
    const uint32_t G = seg_count(n);
    const uint64_t need = flh_schedule_workspace_bytes(n);
    if (workspace_bytes < need) return fl_set_error(FLH_E_ARG, "workspace of %llu bytes, %llu needed for %u chunks", (unsigned long long)workspace_bytes,
                                                        (unsigned long long)need, n);
    if ((uintptr_t)d_workspace % alignof(SegHeader)) return fl_set_error(FLH_E_ARG, "workspace must be %zu-byte aligned", alignof(SegHeader));
    a.seg = (SegHeader*)d_workspace;
    FL_LAUNCH(fl_sched_seg_totals, dim3(G), dim3(kSegBlock), 0, s, a);
    static_assert(kSegChunks == 8 * kWave * 2, "a segment is one pass of fl_schedule_kernel<8, 2>");
    FL_LAUNCH((fl_schedule_kernel<8, 2, true>), dim3(G), dim3(8 * kWave), 0, s, a);
    FL_LAUNCH(fl_sched_seg_finish, dim3(G), dim3(kSegBlock), 0, s, a);
    FL_HIP(hipGetLastError());
    return expand_tiles(p, s);
  }
  if (p->d_table_by_lane && n > 0) return fl_set_error(FLH_E_ARG, "d_table_by_lane needs the uniform closed-form split (no d_sizes, no d_src_off, quantum == chunk_bytes, n_rows <= %d)", kRowCache);
  // one workgroup; more wavefronts first, then more chunks per thread, as the chunk count grows (measured best shapes)
  if ((variant == 0 && n <= kWave && p->n_rows <= 4) || variant == 1) {   // a lone wavefront prefixes four credit rows per turn
    FL_LAUNCH((fl_schedule_kernel<1, 1>), dim3(1), dim3(kWave), 0, s, a);
  } else if ((variant == 0 && n <= 4 * kWave) || variant == 2) {
    FL_LAUNCH((fl_schedule_kernel<4, 1>), dim3(1), dim3(4 * kWave), 0, s, a);
  } else if ((variant == 0 && n <= 8 * kWave) || variant == 3) {
    FL_LAUNCH((fl_schedule_kernel<8, 1>), dim3(1), dim3(8 * kWave), 0, s, a);
  } else if ((variant == 0 && n <= 16 * kWave) || variant == 4) {
    FL_LAUNCH((fl_schedule_kernel<8, 2>), dim3(1), dim3(8 * kWave), 0, s, a);
  } else if ((variant == 0 && n <= 32 * kWave) || variant == 5) {
    FL_LAUNCH((fl_schedule_kernel<8, 4>), dim3(1), dim3(8 * kWave), 0, s, a);
  } else {
    FL_LAUNCH((fl_schedule_kernel<8, 8>), dim3(1), dim3(8 * kWave), 0, s, a);
  }
  FL_HIP(hipGetLastError());
  return expand_tiles(p, s);
}

int flh_schedule(const flh_sched_params* p, void* stream) {
  return schedule_with(p, stream, p ? p->d_workspace : nullptr, p ? p->workspace_bytes : 0);
}

int fl_sched_scratch_resolve(int device) {
  if (device < 0 || device >= kScratchDevices) return fl_set_error(FLH_E_ARG, "device %d has no slot for the scheduler's own workspace (%d devices at most)", device, kScratchDevices);
  if (g_scratch_ptr[device].load(std::memory_order_acquire)) return FLH_OK;
  int current = -1;
  FL_HIP(hipGetDevice(&current));
  if (current != device) return fl_set_error(FLH_E_STATE, "device %d must be current to resolve its copy of the scheduler's workspace (current: %d)", device, current);
  void* ptr = nullptr;
  FL_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));   // this device's copy of the array; `scratch` itself is not an address the host may use
  if (!ptr) return fl_set_error(FLH_E_HIP, "hipGetSymbolAddress returned no address for the scheduler's workspace on device %d", device);
  g_scratch_ptr[device].store(ptr, std::memory_order_release);
  return FLH_OK;
}

int flh_schedule_static(const flh_sched_params* p, void* stream) {
  if (!p) return fl_set_error(FLH_E_ARG, "null params");
  if (p->n_chunks > FLH_SCHED_STATIC_MAX_CHUNKS)
    return fl_set_error(FLH_E_ARG, "%u chunks exceed the %u that the library's own workspace serves; lend one to flh_schedule instead", p->n_chunks,
                        (unsigned)FLH_SCHED_STATIC_MAX_CHUNKS);
  int rc = fl_need_init();
  if (rc) return rc;
  int device = -1;
  FL_HIP(hipGetDevice(&device));
  rc = fl_sched_scratch_resolve(device);   // resolved at flh_init for the device named there; a first call on another device lands here
  if (rc) return rc;
  return schedule_with(p, stream, g_scratch_ptr[device].load(std::memory_order_acquire), kScratchBytes);
}

}  // extern "C"
