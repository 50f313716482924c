/*
 * fuselink_hip.h -- C ABI of the MI355X (gfx950) FuseLink data path.
 *
 * One shared library, libnccl-net-fuselink.so, carries two interfaces:
 *   1. the NCCL/RCCL net-plugin tables declared in fuselink_net.h (what a communication library
 *      dlopen()s), and
 *   2. the entry points below: the chunk -> lane scheduler, the striping / reassembly copy kernels
 *      and the HIP-VMM staging windows that the plugin is built from.  They are exported so a host
 *      runtime (or a test harness) can drive the same path without the plugin's request machinery.
 *
 * Conventions: plain C types only.  Every function returns 0 on success or a negative FLH_E_* code;
 * flh_last_error() returns a thread-local message for the last failure.  Pointers named d_* are
 * device memory on the current HIP device; `stream` is a hipStream_t passed as void* (NULL = the
 * null stream).  Nothing here blocks on the GPU unless its comment says so.
 *
 * Each entry point names the reference code it replaces (paths inside the FuseLink tree).
 */
#ifndef FUSELINK_HIP_H_
#define FUSELINK_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FLH_MAX_LANES     16                      /* MAX_NIC_NUM, src/monitor.h:18 */
#define FLH_UNIT_BYTES    (2u * 1024u * 1024u)    /* BUFFER_UNIT, src/cumem.h:7 */
#define FLH_POOL_UNITS    256                     /* MAX_MEM_TABLE_SIZE, src/cumem.cu:9 */
#define FLH_TILE_BYTES    32768u                  /* default copy tile; must be a multiple of 128 */

#define FLH_OK            0
#define FLH_E_ARG        -1   /* bad argument (shape, alignment, null pointer) */
#define FLH_E_HIP        -2   /* a HIP runtime call failed; message holds hipGetErrorString */
#define FLH_E_NODEV      -3   /* no usable GPU */
#define FLH_E_NOMEM      -4   /* unit pool exhausted (cumem.cu:176-179) */
#define FLH_E_RANGE      -5   /* a chunk would land outside its staging window */
#define FLH_E_STATE      -6   /* object used in the wrong state */

/* One row of the chunk -> lane table (32 bytes, device and host layout identical). */
typedef struct flh_chunk_desc {
  uint64_t src_off;    /* byte offset of the chunk in the user buffer */
  uint64_t win_off;    /* byte offset in its lane's staging window */
  uint32_t len;        /* bytes */
  uint32_t lane;       /* staging window / virtual NIC index */
  uint32_t tile_base;  /* exclusive prefix of ceil(len / tile_bytes): first copy tile of the chunk */
  uint32_t epoch;      /* credit epoch the chunk was scheduled in */
} flh_chunk_desc;

/* Scheduler state carried from one call to the next (device memory, 144 bytes). */
typedef struct flh_sched_state {
  uint64_t epoch_bytes;               /* bytes already scheduled in the current epoch */
  uint64_t chunk_index;               /* global index of the next chunk */
  uint64_t lane_off[FLH_MAX_LANES];   /* next free byte of each staging window */
} flh_sched_state;

/* One copy tile of a table: tile_bytes (the last one of a chunk: fewer) bytes at src_off of the user buffer, at
 * win_off of lane's window; row = the chunk it belongs to. */
typedef struct flh_tile_desc {
  uint64_t src_off;
  uint64_t win_off;
  uint32_t len;
  uint32_t lane;
  uint32_t row;
  uint32_t pad;
} flh_tile_desc;

/* Summary written by the scheduler next to the table (device memory, 216 bytes). */
typedef struct flh_sched_hdr {
  uint64_t total_bytes;
  uint32_t total_tiles;
  uint32_t n_chunks;
  uint32_t flags;                      /* FLH_SCHED_F_* */
  uint32_t uniform_tiles;              /* tiles per chunk if the split is uniform (d_sizes == NULL), else 0 */
  uint64_t lane_bytes[FLH_MAX_LANES];  /* bytes this call put on each lane */
  uint32_t lane_chunks[FLH_MAX_LANES]; /* chunks this call put on each lane */
} flh_sched_hdr;

#define FLH_SCHED_F_NO_CREDIT 1u       /* some epoch had all-zero credits: static lane policy used */

/* flh_sched_params.mode */
#define FLH_SCHED_RESET_OFFSETS 1u     /* start every lane at window offset 0 instead of the state's */
#define FLH_SCHED_NEW_EPOCH     4u     /* start with zero epoch bytes instead of the state's (credits were refreshed) */
#define FLH_SCHED_MIRROR        2u     /* win_off = src_off: each window mirrors the user buffer, the
                                          reference's translation window + (data - start_addr)
                                          (src/plugin.cc:1582, 1626); windows must be bound that far */

typedef struct flh_sched_params {
  const uint32_t* d_sizes;     /* n chunk sizes, or NULL for the uniform split of total_bytes */
  uint64_t total_bytes;        /* used when d_sizes == NULL */
  uint32_t chunk_bytes;        /* used when d_sizes == NULL */
  const uint64_t* d_src_off;   /* n explicit source offsets, or NULL for src_base + running sum */
  uint64_t src_base;
  uint32_t n_chunks;
  uint32_t n_lanes;            /* 1..16 */
  const uint32_t* d_credits;   /* n_rows x n_lanes credit table; NULL = the single row in inline_credits */
  uint32_t n_rows;             /* >= 1; epoch e reads row e mod n_rows */
  uint32_t epoch_len;          /* chunks per credit epoch; 0 = a single epoch */
  uint64_t quantum;            /* bytes per credit (the nominal chunk size) */
  uint32_t tile_bytes;         /* copy tile the table is partitioned for (multiple of 128) */
  uint32_t mode;               /* FLH_SCHED_* bits */
  flh_sched_state* d_state;    /* in/out, or NULL to start from zero and discard */
  flh_chunk_desc* d_table;     /* out: n_chunks rows */
  flh_sched_hdr* d_hdr;        /* out */
  uint32_t inline_credits[FLH_MAX_LANES]; /* one credit row passed by value (used when d_credits == NULL) */
  flh_chunk_desc* d_table_by_lane; /* optional out: the same n_chunks rows in destination order -- grouped by lane,
                                      chunk order kept inside a lane, the last chunk's lane last, tile_base =
                                      position * tiles per chunk.  flh_stripe driven by this copy writes every
                                      window front to back, which is faster once a message exceeds the Infinity
                                      Cache.  Uniform closed-form split only (d_sizes == NULL, d_src_off == NULL,
                                      quantum == chunk_bytes, n_rows <= 32); FLH_E_ARG otherwise. */
  struct flh_tile_desc* d_tiles; /* optional out: the table expanded to one descriptor per copy tile (a second launch
                                    behind the scheduler's), for flh_stripe_tiles / flh_reassemble_tiles: a copy
                                    workgroup then reads one descriptor instead of searching the table for its row,
                                    which pays from a few thousand rows of unequal size on */
  uint32_t tiles_cap;          /* descriptors d_tiles holds; total_bytes / tile_bytes + n_chunks always suffices */
  uint32_t pad_;
  void* d_workspace;           /* optional: flh_schedule_workspace_bytes(n_chunks) bytes of 8-byte aligned device memory; with it a
                                  chunk list of 4096 chunks or more that needs the scan (d_sizes, d_src_off or
                                  quantum != chunk_bytes) is scheduled by one workgroup per 1024 chunks in three
                                  launches instead of by one workgroup; same table, header and state */
  uint64_t workspace_bytes;
  uint32_t wave_chunks;        /* uniform closed-form split only: the windows are reused every wave_chunks chunks, so a
                                  row's win_off counts from the first chunk of its wave on an empty window -- the rows
                                  [w * wave_chunks, (w + 1) * wave_chunks) are the table of wave w as a call for that
                                  wave alone (RESET_OFFSETS, state carried) would write it.  Header and state are the
                                  whole call's.  0 = one wave.  One scheduler launch then serves a message that moves
                                  through windows smaller than itself (src/cumem.cu:9: a 512 MiB pool). */
  uint32_t pad2_;
} flh_sched_params;

/* ---- library ------------------------------------------------------------------------------ */
/* Selects `device`, checks that it is a gfx950 part, loads kernel attributes.  Idempotent. */
int flh_init(int device);
const char* flh_last_error(void);
/* bytes of flh_sched_params.d_workspace that flh_schedule needs for n_chunks chunks */
uint64_t flh_schedule_workspace_bytes(uint32_t n_chunks);
/* compile-time facts: 0 tile bytes, 1 max lanes, 2 unit bytes, 3 pool units, 4 sizeof(desc),
 * 5 sizeof(state), 6 sizeof(hdr), 7 ABI version, 8 sizeof(flh_windows), 9 sizeof(flh_sched_params),
 * 10 sizeof(flh_batch_params) */
int64_t flh_constant(int which);
/* Launch tunables, for experiments (no counterpart in the reference): "grid_per_cu" = copy
 * workgroups launched per compute unit (0 = one per tile), "nontemporal" = 0/1 streaming loads and
 * stores everywhere / nowhere (-1, the default: per side -- user buffers stream once a launch moves 16 (written side) or 128 MiB (read side),
 * the staging windows stay cacheable until a message passes 256 MiB and they outgrow the Infinity Cache).
 * "stream_mode_out" / "stream_mode_in" = 0..3 force the mode of the striping / reassembly side (bit 0 loads,
 * bit 1 stores; -1 = the policy).  "stream_mode_deliver" = the same for flh_stage_deliver_*, with bit 4 for the stores into
 * the windows (-1: loads and window stores as the striping side's, the other stores as the reassembly side's).
 * "stripe_dest_order" = 0/1: flh_stripe_uniform walks the chunks lane by lane, so that every window is written
 * front to back (-1 = only for messages past 256 MiB, whose windows no longer fit the Infinity Cache, the default).
 * "sched_seg_min" = chunks from which a lent workspace makes the scan scheduler use several workgroups (4096).
 * "xcd_runs" = 1/0: launches of 256 copy workgroups and more hand each of the eight XCDs runs of 32 consecutive
 * tiles (1 MiB) instead of every eighth tile (1, the default; 3-5 % faster copies).
 * "lane_share1_tiles" = lane-engine batches of up to this many copy tiles are handed to the workers one tile at a time
 * (latency), larger ones two neighbouring tiles at a time (throughput); -1 = three quarters of the engine's workers,
 * the default.
 * Test hooks (refused with FLH_E_STATE unless the environment holds NCCL_FUSELINK_TEST_HOOKS=1):
 * "engine_wait_us" = limit of every wait inside a lane engine created afterwards (2 000 000; tests of the failure
 * path ask for a microsecond).
 * "engine_inject_fault" = 1: a lane engine that is started (or started again after idling) while this is set reports
 * a wait that ran out in place of executing its first batch and goes down, every workgroup leaving as after a real
 * one (0; for tests of the failure path, which cannot count on a healthy GPU to miss a limit).
 * "engine_fail_start" = 1: starting the resident kernel fails as a refused launch would (0; the submit that needed the
 * start must then return its error with the batch taken back out of the ring).
 * "engine_trace" = 1: lane engines created afterwards stamp every batch's stages with the GPU's wall clock
 * (flh_engine_trace; 0).
 * The same values can be preset with NCCL_FUSELINK_GRID_PER_CU / NCCL_FUSELINK_NONTEMPORAL.
 * The tunables are process-wide and read by every launch: set them while no other thread launches. */
int flh_tune(const char* key, int64_t value);
/* Per-kernel timing for measurement code (no counterpart in the reference).  Between
 * flh_prof_begin and flh_prof_end every launch this thread makes through the library carries its
 * own start/stop HIP events that bracket the kernel alone; the launches stay asynchronous.
 * flh_prof_end waits for them and returns how many were recorded, filling up to `max` durations
 * (microseconds) and the entry point that launched each: 1 schedule, 2 stripe, 3 reassemble,
 * 4 gather, 5 scatter, 6 copy, 7 stage + deliver.  Launches beyond `capacity` are not timed. */
int flh_prof_begin(int capacity);
int flh_prof_end(double* us_out, int* kernel_out, int max);

/* ---- scheduler ------------------------------------------------------------------------------
 * Replaces FuseLinkConnManager::refreshRxComm / bidTxChannel (src/fuselink.h:153-156, 230-238) and
 * the idle-NIC query behind them (src/monitor.h:191-224) with one kernel launch over a whole send
 * set: an epoch-segmented wavefront prefix scan of the chunk sizes gives each chunk its quantum
 * slot, the credit row of its epoch maps the slot to a lane, and a per-lane scan gives its offset
 * in that lane's staging window.  Equal credits and quantum-sized chunks reproduce the reference's
 * live policy lane = index mod lanes (src/fuselink.h:235). */
int flh_schedule(const flh_sched_params* p, void* stream);

/* flh_schedule for callers that cannot allocate and cannot lend a workspace (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same parameters, table, header
 * and state as flh_schedule; p->d_workspace / p->workspace_bytes are ignored, and a chunk list long enough for the scan over
 * several workgroups uses a workspace of the library's own instead: a static device array of about 224 KiB that every GPU
 * the library runs on holds until the process ends, which serves lists of up to FLH_SCHED_STATIC_MAX_CHUNKS chunks
 * (more: FLH_E_ARG, lend a workspace to flh_schedule).  The call allocates and frees nothing.  All calls on one GPU
 * share that GPU's array: two calls that overlap on one GPU (different streams, or threads) race; calls in stream
 * order on one stream are safe, every launch rewrites what it reads. */
#define FLH_SCHED_STATIC_MAX_CHUNKS (1u << 20)
int flh_schedule_static(const flh_sched_params* p, void* stream);

/* ---- striping / reassembly --------------------------------------------------------------------
 * flh_stripe replaces the send side of ncclIbMultiSend (src/plugin.cc:1467-1495: per-request split,
 * RDMA write out of the staged copy at flmr->addr[dev] + (data - start_addr), src/plugin.cc:1582):
 * every chunk of the table is copied from d_src + src_off into window[lane] + win_off.
 * flh_reassemble replaces the landing of those writes in the receiver's translated buffer
 * (src/plugin.cc:1626): window[lane] + win_off is copied to d_dst + src_off.
 * d_hdr->total_tiles sizes the work; win_cap[l] is the mapped size of window l and a chunk that
 * would cross it is skipped and reported through *d_status (FLH_E_RANGE), never written.
 * n_chunks_max bounds the table rows the kernel may read.  h_hdr is optional: a HOST copy of the
 * header whose total_tiles, n_chunks and uniform_tiles the caller already knows (for a uniform
 * split they follow from the sizes alone); with it the kernel does not wait for d_hdr. */
typedef struct flh_windows {
  void*    base[FLH_MAX_LANES];
  uint64_t cap[FLH_MAX_LANES];
  uint32_t n_lanes;
  uint32_t pad;
} flh_windows;

int flh_stripe(const void* d_src, uint64_t src_bytes, const flh_windows* win,
               const flh_chunk_desc* d_table, const flh_sched_hdr* d_hdr, const flh_sched_hdr* h_hdr,
               uint32_t n_chunks_max, uint32_t tile_bytes, int32_t* d_status, void* stream);
int flh_reassemble(void* d_dst, uint64_t dst_bytes, const flh_windows* win,
                   const flh_chunk_desc* d_table, const flh_sched_hdr* d_hdr, const flh_sched_hdr* h_hdr,
                   uint32_t n_chunks_max, uint32_t tile_bytes, int32_t* d_status, void* stream);

/* The same pair driven by the per-tile descriptors that flh_schedule wrote to d_tiles (tiles_cap entries).  The
 * number of tiles comes from h_hdr when given, else from d_hdr; a table with more tiles than tiles_cap is refused
 * through *d_status (FLH_E_RANGE), and so is a descriptor that would leave the buffer or its window.  Like the
 * scheduler itself these have no counterpart in the reference, whose transport posts one contiguous buffer per
 * request (src/plugin.cc:1467-1495). */
int flh_stripe_tiles(const void* d_src, uint64_t src_bytes, const flh_windows* win, const flh_tile_desc* d_tiles,
                     uint32_t tiles_cap, const flh_sched_hdr* d_hdr, const flh_sched_hdr* h_hdr, int32_t* d_status, void* stream);
int flh_reassemble_tiles(void* d_dst, uint64_t dst_bytes, const flh_windows* win, const flh_tile_desc* d_tiles,
                         uint32_t tiles_cap, const flh_sched_hdr* d_hdr, const flh_sched_hdr* h_hdr, int32_t* d_status, void* stream);

/* Scheduler and copy in one launch, for a uniform split (R1) under a single credit row with
 * quantum == chunk_bytes and window offsets starting at 0 -- the shape of every request the plugin
 * issues.  Each workgroup derives its chunk's lane and window offset from the closed form of the
 * schedule instead of reading a table row; flh_stripe_uniform also writes the table and header (when
 * the pointers are given), bit-identical to what flh_schedule produces for the same inputs with
 * FLH_SCHED_RESET_OFFSETS, state {epoch_bytes, 0, ...} and d_sizes == NULL.  Replaces, in one step,
 * the lane choice (src/fuselink.h:230-238) and the send / landing of src/plugin.cc:1467-1495, 1582, 1626.
 * At most 65535 chunks per call. */
typedef struct flh_uniform_params {
  uint64_t total_bytes;
  uint64_t src_base;          /* byte offset of chunk 0 in the user buffer */
  uint64_t epoch_bytes;       /* bytes already scheduled in the current credit epoch (0 after a refresh) */
  uint32_t chunk_bytes;       /* chunk size = quantum */
  uint32_t n_lanes;
  uint32_t tile_bytes;
  uint32_t pad;
  uint32_t credits[FLH_MAX_LANES];
  /* Completion of the reassembly / scatter launch, for callers that poll instead of synchronising (all optional; the
   * striping side ignores them; no counterpart in the reference, whose completions come from the NIC's queue,
   * src/plugin.cc:1801-1955).
   * d_done_word: a host-visible word (e.g. pinned, mapped memory).  The launch counts its finished workgroups in
   * *d_done_count (device memory, zero before the first use; the kernel leaves it zero) and the last of them stores
   * done_value to *d_done_word with release semantics at system scope, after every workgroup's stores: a thread that
   * reads done_value there with acquire semantics may use the destination buffer.  Launches that share a count word
   * must be ordered (one stream).
   * done_event: a hipEvent_t that the launch's kernel completes (hipEventQuery then answers for the kernel), which
   * spares the separate packet of a hipEventRecord behind it.
   * d_start_word (striping / gather side only): a host-visible word to which the launch's first workgroup stores
   * start_value as it starts.  Work on a stream runs in order, each kernel after everything before it has finished
   * and its results are visible on the device, so a caller that numbers its launches learns from the word that all
   * launches before this one are complete.  The cheapest of the three: one store per launch, but it only says so once
   * a later launch has begun. */
  uint32_t* d_done_word;
  uint32_t* d_done_count;
  uint32_t done_value;
  uint32_t start_value;
  void* done_event;
  uint32_t* d_start_word;
} flh_uniform_params;

int flh_stripe_uniform(const void* d_src, uint64_t src_bytes, const flh_windows* win,
                       const flh_uniform_params* u, flh_chunk_desc* d_table_out,
                       flh_sched_hdr* d_hdr_out, int32_t* d_status, void* stream);
int flh_reassemble_uniform(void* d_dst, uint64_t dst_bytes, const flh_windows* win,
                           const flh_uniform_params* u, int32_t* d_status, void* stream);
/* flh_stripe_uniform for a sender whose receiver is not this process: the workgroup that stages a tile in its
 * lane's window writes it, from the same registers, into the same lane and offset of `landing` as well, windows of the
 * receiver (its device memory, opened here), which plays the part of the lane's NIC in the reference -- the RDMA write
 * out of the staged copy into the receiver's translated buffer (src/plugin.cc:1453-1495, 1582, 1626).  The receiver
 * runs flh_reassemble_uniform over its landing windows with the same parameters.  landing->cap bounds the carry as
 * win->cap bounds the staging (FLH_E_RANGE through *d_status; a chunk that would leave either window is written to
 * neither).  The completion fields of `u` (done word / event) report this launch, which is the
 * last of the path on the sending side. */
int flh_stripe_uniform_carry(const void* d_src, uint64_t src_bytes, const flh_windows* win, const flh_windows* landing,
                             const flh_uniform_params* u, flh_chunk_desc* d_table_out, flh_sched_hdr* d_hdr_out,
                             int32_t* d_status, void* stream);
/* flh_stripe_uniform + flh_reassemble_uniform in one launch, for a sender that can write the receive buffer itself
 * (the receiver is this process, or a process whose registered buffer is mapped here): every workgroup loads its tile
 * of the message once and stores it twice, into its lane's staging window -- table, header and staged bytes are those
 * of flh_stripe_uniform -- and at the same offset of d_dst as the tile has in d_src, which is where the reference's
 * RDMA write out of the staged copy lands (src/plugin.cc:1453-1495: remote_addr + offset).  A chunk that would leave its
 * window, the source or d_dst (dst_bytes) is written nowhere (FLH_E_RANGE through *d_status).  The completion fields of
 * `u` report this launch. */
int flh_stage_deliver_uniform(const void* d_src, uint64_t src_bytes, void* d_dst, uint64_t dst_bytes, const flh_windows* win,
                              const flh_uniform_params* u, flh_chunk_desc* d_table_out, flh_sched_hdr* d_hdr_out,
                              int32_t* d_status, void* stream);

/* Several requests in one launch: requests that are waiting together -- NCCL keeps up to NCCL_STEPS = 8 in flight per
 * channel (src/fuselink.h:14) and runs several channels to a peer, which all share the per-NIC lane comms
 * (src/fuselink.h:271-272, src/plugin.cc:727-753) -- are scheduled and copied by ONE launch per direction, so the
 * launch cost is paid once per batch instead of once per request.  No counterpart in the reference, which posts one
 * RDMA write per request.
 *
 * The requests form 1..FLH_SEG_MAX segments, in order.  A segment is a run of requests that is scheduled as ONE
 * message -- the concatenation of its buffers -- from its own credit-epoch prefix under its own credit row, exactly as
 * flh_stripe_uniform schedules a message: the requests of one connection between two lane-decision refreshes.  Every
 * request of a segment but its last must be a whole number of chunks.  In the staging windows the segments follow each
 * other: on every lane, segment k starts where segment k - 1 ended, rounded up to 128 bytes (the alignment of the
 * reference's per-QP pieces, src/plugin.cc:1467).  n_seg == 0 stands for one segment of all requests under u.credits
 * and u.epoch_bytes.  u.total_bytes must equal the sum of bytes[]; u.src_base is ignored; a credit row must sum below
 * 2^32.
 *
 * Table rows (flh_stripe_batch, when d_table_out is given) are those of each segment's message -- src_off counts from
 * the segment's first byte -- with the segment's lane base added to win_off and tile_base counted over the whole
 * launch; the header holds the totals of the launch. */
#define FLH_BATCH_MAX 32
#define FLH_SEG_MAX 8
typedef struct flh_batch_segment {
  uint64_t epoch_bytes;       /* bytes already scheduled in the segment's credit epoch (0 after a refresh) */
  uint32_t n_req;             /* requests of the batch, in order, that form this segment */
  uint32_t pad;
  uint32_t credits[FLH_MAX_LANES];
} flh_batch_segment;
typedef struct flh_batch_params {
  flh_uniform_params u;
  uint32_t n_req;             /* 1..FLH_BATCH_MAX */
  uint32_t n_seg;             /* 0 (one segment, u.credits / u.epoch_bytes) or 1..FLH_SEG_MAX */
  const void* d_src[FLH_BATCH_MAX];
  void*       d_dst[FLH_BATCH_MAX];
  uint64_t    bytes[FLH_BATCH_MAX];
  flh_batch_segment seg[FLH_SEG_MAX];
} flh_batch_params;

int flh_stripe_batch(const flh_batch_params* b, const flh_windows* win, flh_chunk_desc* d_table_out,
                     flh_sched_hdr* d_hdr_out, int32_t* d_status, void* stream);
int flh_reassemble_batch(const flh_batch_params* b, const flh_windows* win, int32_t* d_status, void* stream);
/* flh_stripe_batch + flh_reassemble_batch in one launch, as flh_stage_deliver_uniform: request q's bytes go into the
 * windows and into b->d_dst[q]. */
int flh_stage_deliver_batch(const flh_batch_params* b, const flh_windows* win, flh_chunk_desc* d_table_out,
                            flh_sched_hdr* d_hdr_out, int32_t* d_status, void* stream);
/* flh_stripe_batch with the carry of flh_stripe_uniform_carry (b->d_dst is not used). */
int flh_stripe_batch_carry(const flh_batch_params* b, const flh_windows* win, const flh_windows* landing,
                           flh_chunk_desc* d_table_out, flh_sched_hdr* d_hdr_out, int32_t* d_status, void* stream);
/* Where the batch leaves every staging window: lane_end[l] = first free byte of lane l after the last segment
 * (host arithmetic, nothing is launched); seg_base, if given, receives FLH_SEG_MAX x FLH_MAX_LANES lane bases, row k
 * those of segment k.  A caller sizes its batches with it so that no lane outgrows its window. */
int flh_batch_layout(const flh_batch_params* b, uint64_t* lane_end, uint64_t* seg_base);
/* ---- lane engine: batches without a launch per batch ------------------------------------------------------------
 * A resident kernel -- one dispatcher workgroup, the others workers, by default one worker per two compute units -- that
 * executes batches as flh_stripe_batch + flh_reassemble_batch would, but takes them from a descriptor ring in pinned
 * host memory instead of from kernel launches: flh_engine_submit writes the descriptor and advances a tail word (about
 * a microsecond of host time instead of about ten for a launch pair), the engine stripes every tile into the windows
 * and, from the registers it staged the tile from, writes it on into the receive buffer (nothing is read back: what
 * the windows hold and what is received are the same loaded bytes), and stores the batch's number to a host-visible
 * word when its last workgroup has left the batch (flh_engine_completed reads it: no call into the runtime).  Rows,
 * header, staged bytes and received bytes are those of the launched pair.  Several batches are in flight at once, so successive batches must not share staging
 * windows: the caller rotates window_sets (1..8) sets of windows, batch number k taking set (k - 1) mod window_sets, and
 * the engine lets a batch in only once batch k - window_sets is complete.  With nothing to do for idle_us (default 200) the
 * engine goes down and the next submit starts it again with one launch.  Every wait inside the kernel is bounded;
 * flh_engine_error reports FLH_E_STATE if one ran out.  No counterpart in the reference, whose NIC plays this part.
 * flh_engine_submit and flh_engine_destroy are not thread-safe (one submitter at a time); the readers are. */
typedef struct flh_engine flh_engine;
int flh_engine_create(int device, uint32_t workgroups, uint32_t idle_us, uint32_t window_sets, flh_engine** out);
/* *seq_out = the batch's number, from 1; seg_base_out (optional) = the lane bases of its segments, as flh_batch_layout gives them */
int flh_engine_submit(flh_engine* e, const flh_batch_params* b, const flh_windows* win, flh_chunk_desc* d_table_out,
                      flh_sched_hdr* d_hdr_out, int32_t* d_status, uint64_t* seq_out, uint64_t* seg_base_out);
/* The two halves of a batch whose ends are different processes, numbered, ordered and reported like any other batch of
 * the engine.  FLH_ENGINE_SEND: stripe into `win` (the caller's rotating sets, as for flh_engine_submit) and write every
 * tile into the same lane and offset of `landing` as well, as flh_stripe_batch_carry does; b->d_dst is not used.  FLH_ENGINE_RECV: reassemble out of `win`
 * -- the landing windows a sender has filled -- into b->d_dst; b->d_src, `landing` (NULL) and the table pointers are not
 * used.  A batch is complete when its bytes are in memory: the landing windows' for a send, the receive buffers' for a
 * receive.  Stands where the reference's NIC stands on either side (src/plugin.cc:1453-1495 / 1616-1677). */
#define FLH_ENGINE_LOOP 0u   /* what flh_engine_submit submits: both ends in this process */
#define FLH_ENGINE_SEND 1u
#define FLH_ENGINE_RECV 2u
int flh_engine_submit_wire(flh_engine* e, uint32_t kind, const flh_batch_params* b, const flh_windows* win, const flh_windows* landing,
                           flh_chunk_desc* d_table_out, flh_sched_hdr* d_hdr_out, int32_t* d_status, uint64_t* seq_out, uint64_t* seg_base_out);
/* How long the resident kernel stays although work keeps coming (microseconds; 0 = as long as there is work; default
 * 1000).  A kernel that never ends holds its hardware queue; the runtime puts several streams on one queue when a process
 * has more streams than queues, and what it has queued behind the engine waits until the engine leaves.  With a bound
 * the engine leaves between two batches when its time is up, and the next flh_engine_submit -- or flh_engine_poke, for a
 * caller with batches outstanding and nothing further to submit -- starts it again.  flh_engine_needs_start says
 * whether flh_engine_poke would start it (two loads of host memory).  flh_engine_poke is not thread-safe against
 * flh_engine_submit. */
int flh_engine_set_resident(flh_engine* e, uint32_t resident_us);
/* Measurement (no counterpart in the reference): where the batches first_seq .. first_seq + n - 1 (numbers as
 * flh_engine_submit returned them, all complete, among the last 1024) spent their time inside the resident kernel.
 * FLH_ENGINE_STAMPS values of the GPU's 100 MHz wall clock per batch: the dispatcher saw the host's tail beyond the
 * batch; it published the batch to the workers; the worker with the first share saw that; it was let in (the batch
 * whose windows this one reuses was complete); it had the descriptor; it had moved its shares (their stores in
 * memory); the last worker out had the completion word's store acknowledged.  Only for an engine created while flh_tune("engine_trace") was set (FLH_E_STATE otherwise);
 * synchronous (a device-to-host copy). */
#define FLH_ENGINE_STAMPS 7
int flh_engine_trace(flh_engine* e, uint64_t first_seq, uint32_t n, uint64_t* stamps_out);
int flh_engine_needs_start(const flh_engine* e);
int flh_engine_poke(flh_engine* e);
uint64_t flh_engine_completed(const flh_engine* e);   /* batches complete: all with a number up to this one */
int flh_engine_error(const flh_engine* e);
uint64_t flh_engine_launches(const flh_engine* e);    /* engine kernels started so far */
int flh_engine_destroy(flh_engine* e);                /* asks the engine down and waits for it */

/* Paged variants for non-contiguous sources (KV-cache blocks, src/experiments/serving/model.hh:
 * 198-201 gives the page shape): a chunk whose row says src_off stands for the pages
 * d_page_table[src_off / page_bytes ...] (pages_per_chunk of them) of a pool of page_bytes-sized
 * pages -- for the uniform split from src_base = 0 that is d_page_table[c*pages_per_chunk ...] for
 * chunk c; gather packs them into the chunk's window slot, scatter puts them back at the same page
 * numbers of d_pool.  The rows may come in any order (d_table_by_lane for the gather); src_off must
 * be a multiple of page_bytes and below n_chunks*pages_per_chunk pages, else FLH_E_RANGE is
 * reported through *d_status.  use_lds != 0 stages each tile through LDS. */
int flh_gather_pages(const void* d_pool, uint64_t pool_pages, const uint32_t* d_page_table,
                     uint32_t page_bytes, uint32_t pages_per_chunk, const flh_windows* win,
                     const flh_chunk_desc* d_table, uint32_t n_chunks, int use_lds,
                     int32_t* d_status, void* stream);
int flh_scatter_pages(void* d_pool, uint64_t pool_pages, const uint32_t* d_page_table,
                      uint32_t page_bytes, uint32_t pages_per_chunk, const flh_windows* win,
                      const flh_chunk_desc* d_table, uint32_t n_chunks, int use_lds,
                      int32_t* d_status, void* stream);

/* The paged pair with the scheduler folded in, as flh_stripe_uniform / flh_reassemble_uniform do for a flat buffer:
 * the message of u->total_bytes bytes is the pages d_page_table[0 .. ceil((src_base + total_bytes) / page_bytes)) of
 * the pool, in that order; no table has to exist, the gather writes it to d_table_out / d_hdr_out (may be NULL).
 * u->tile_bytes must divide page_bytes (a copy tile never straddles a page); u->chunk_bytes and u->src_base must be
 * multiples of page_bytes.  A page number beyond pool_pages reports FLH_E_RANGE through *d_status.  No counterpart in
 * the reference; the page shape is the serving experiment's KV block (experiments/serving/model.hh:198-201). */
int flh_gather_pages_uniform(const void* d_pool, uint64_t pool_pages, const uint32_t* d_page_table, uint32_t page_bytes,
                             const flh_windows* win, const flh_uniform_params* u, flh_chunk_desc* d_table_out,
                             flh_sched_hdr* d_hdr_out, int32_t* d_status, void* stream);
int flh_scatter_pages_uniform(void* d_pool, uint64_t pool_pages, const uint32_t* d_page_table, uint32_t page_bytes,
                              const flh_windows* win, const flh_uniform_params* u, int32_t* d_status, void* stream);

/* Plain device copy with the same inner loop as the striping kernels (roofline calibration). */
int flh_copy(void* d_dst, const void* d_src, uint64_t bytes, void* stream);
/* Up to FLH_MAX_LANES independent runs in one launch: run r moves bytes[r] from d_src[r] to d_dst[r] (empty runs are
 * skipped).  It carries the staged bytes of every lane from a sender's windows into a receiver's, the part a NIC
 * per lane plays in the reference (one RDMA write per lane comm, src/plugin.cc:1453-1495). */
int flh_copy_runs(void* const* d_dst, const void* const* d_src, const uint64_t* bytes, uint32_t n, void* stream);

/* ---- R2: request -> QP pieces (src/plugin.cc:1467-1495), host arithmetic ------------------------ */
int flh_qp_split(int size, int nqps, int* off, int* len);

/* ---- staging windows on HIP VMM ------------------------------------------------------------------
 * Replaces the 2 MiB slot pool of src/cumem.cu (init_cumem 29-57, register_cumem 107-184,
 * remap_cumem 72-105, free_cumem 60-70) and the per-device windows of FuseLinkMemRegionInit
 * (src/fuselink.cc:4-59).  A pool owns `units` physical 2 MiB allocations (hipMemCreate); a window
 * is a virtual range (hipMemAddressReserve) whose leading units are bound to pool slots first-fit
 * (hipMemMap + hipMemSetAccess).  Unlike the reference, errors come back as codes, not exit(1)
 * (src/checks.h:17-23). */
typedef struct flh_pool flh_pool;
typedef struct flh_window flh_window;

int flh_pool_create(int device, uint32_t units, flh_pool** out);
int flh_pool_destroy(flh_pool* pool);             /* all windows must be destroyed first */
int flh_pool_free_units(const flh_pool* pool);    /* number of unbound slots */
int flh_pool_slot_of(const flh_pool* pool, const void* va); /* ptr2dev analogue (cumem.cu:186-193) */
uint64_t flh_pool_granularity(const flh_pool* pool);

int flh_window_create(flh_pool* pool, uint64_t va_bytes, flh_window** out);
/* grow the bound prefix to cover at least `bytes` (rounded up to units); FLH_E_NOMEM if the pool
 * cannot supply them (slots bound before the failure stay bound, as in cumem.cu:176-179) */
int flh_window_bind(flh_window* w, uint64_t bytes);
/* unbind the trailing units so that at most `bytes` stay bound (0 = all); slots return to the pool */
int flh_window_trim(flh_window* w, uint64_t bytes);
int flh_window_destroy(flh_window* w);
void* flh_window_base(const flh_window* w);
uint64_t flh_window_bound_bytes(const flh_window* w);
/* slot ids backing the first `max` units, in order; returns the number of bound units */
int flh_window_slots(const flh_window* w, int* slots, int max);
/* DMA-BUF file descriptor for one bound staging unit of the window (`offset` a multiple of the unit, `bytes`
 * exactly one unit: a descriptor covers one physical allocation): what a NIC driver registers so that it can read a lane's staged data, the
 * counterpart of the reference handing `fd`/`offset` to ibv_reg_dmabuf_mr for every relay buffer
 * (src/plugin.cc:1278-1280).  The caller closes the descriptor. */
int flh_window_export_dmabuf(const flh_window* w, uint64_t offset, uint64_t bytes, int* fd_out);

/* ---- regions: the regMr-time object (src/plugin.cc:1168-1330, 1337-1408; src/fuselink.h:39-52) ---
 * One region per base allocation, shared and reference-counted by base address; it owns one
 * staging window per lane.  flh_region_translate is the reference's pointer translation
 * window_base + (data - start_addr) (src/plugin.cc:1582, 1626). */
typedef struct flh_region flh_region;
/* n_lanes may be 0: the region then only keeps the registration (base, size, reference count). */
int flh_region_acquire(flh_pool* pool, void* base, uint64_t bytes, uint32_t n_lanes,
                       uint64_t bound_bytes_per_lane, flh_region** out);
int flh_region_release(flh_region* r);            /* returns remaining refs (>= 0) or an error */
int flh_region_refs(const flh_region* r);
int flh_region_windows(const flh_region* r, flh_windows* out);
void* flh_region_translate(const flh_region* r, uint32_t lane, const void* data);

#ifdef __cplusplus
}
#endif
#endif /* FUSELINK_HIP_H_ */
