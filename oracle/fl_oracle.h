/*
 * fl_oracle.h -- CPU restatement of FuseLink's chunking / lane / staging arithmetic.
 *
 * TEST INFRASTRUCTURE ONLY.  This is the checker the GPU path is compared against.
 * Nothing that ships (the HIP library, the net plugin, the Python host mirror) may
 * include, link or call it; only tests/, the smoke check and the bench's CPU-baseline
 * leg do.
 *
 * Every function cites the reference lines it follows (paths under the FuseLink tree).
 * Pinning status of each function (what, other than this file, fixes its result):
 *
 *   fl_split_*        closed form of NCCL 2.19.4's step split (submodule not vendored in the
 *                     reference tree) -- hand vectors + invariants.  PARITY UNPINNED against
 *                     NCCL's own code; pinned against the closed form only.
 *   fl_qp_split       plugin.cc:1467-1495 -- hand vectors, invariants.
 *   fl_lane_static    fuselink.h:235 -- brute force.
 *   fl_refresh_*      plugin.cc:38,1443,1700 -- index-set closed form.
 *   fl_mon_*          monitor.h:191-250, monitor.cpp:159-193 -- checked against the reference's
 *                     own MonitorClient compiled from monitor.h (oracle/_ref) for mark / pick /
 *                     status and the shared-memory layout; the daemon tick (monitor.cpp needs
 *                     libibverbs headers, absent) is restated and pinned by hand vectors.
 *   fl_tx_usage_mask / fl_rx_credits_from_status  build-defined content of a reference placeholder
 *                     (fuselink.h:261-267) -- hand vectors; all-idle gives the placeholder's 0xffffffff; an all-ones
 *                     mask reduces to fl_credits_from_status; brute force over every status pattern of 4 lanes.
 *   fl_credit_schedule  build-defined (the reference has no weighted scheduler); pinned by the
 *                     five properties listed at its declaration and brute force on tiny inputs.
 *   fl_table_by_lane  build-defined reordering of a finished table (destination order for the striping
 *                     kernel) -- pinned by a stable sort in numpy and the permutation invariants.
 *   fl_align_up / fl_window_layout / fl_translate / fl_relay_gpu / fl_page_span
 *                     fuselink.cc:15-40, plugin.cc:1181-1201,1582,1626 -- closed forms.
 *   fl_pool_*         cumem.cu:107-184 -- bitmap model, exhaustion at slot 257.
 *   fl_reqtab_* / fl_fifo_*  plugin.cc:1070-1090,1510-1517,1632 -- hand vectors.
 */
#ifndef FL_ORACLE_H_
#define FL_ORACLE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- constants restated from the reference -------------------------------------------- */
#define FLO_MAX_GPU_NUM        8      /* fuselink.h:12 */
#define FLO_STEPS              8      /* fuselink.h:14 (mirrors NCCL_STEPS) */
#define FLO_MAX_NIC_NUM        16     /* monitor.h:18 */
#define FLO_NNIC_PER_GROUP     1      /* monitor.h:19 */
#define FLO_NGROUP             (FLO_MAX_NIC_NUM / FLO_NNIC_PER_GROUP) /* monitor.h:20 */
#define FLO_MONITOR_TIMEOUT_US 160    /* monitor.h:26 */
#define FLO_BUFFER_UNIT        (2u * 1024u * 1024u) /* cumem.h:7 */
#define FLO_MAX_MEM_TABLE_SIZE 256    /* cumem.cu:9 */
#define FLO_N_FINISHED_BATCH   8      /* plugin.cc:38 */
#define FLO_MAX_REQUESTS       256    /* plugin.cc:382 (32 * 8) */
#define FLO_MAX_RECVS          8      /* plugin.cc:358 */
#define FLO_QP_ALIGN           128    /* plugin.cc:1468 */

#define FLO_NIC_IDLE     0            /* monitor.h:40-44 */
#define FLO_NIC_BUSY     1
#define FLO_NIC_BORROWED 2

/* ---- R1: message -> chunks (NCCL proxy step split; closed form) ------------------------ */
/* n = ceil(N / C); off_i = i*C; len_i = min(C, N - i*C).  Operating point of the reference:
 * NCCL_BUFFSIZE / FUSELINK_STEPS = 4 MiB / 8 = 512 KiB (run_bw_test.sbatch:21,34; fuselink.h:14). */
uint64_t fl_split_count(uint64_t nbytes, uint32_t chunk);
void     fl_split_get(uint64_t nbytes, uint32_t chunk, uint64_t i, uint64_t* off, uint32_t* len);
/* NCCL step size = buffsize / steps (fuselink.h:14; run_bw_test.sbatch:21). */
uint32_t fl_step_size(uint64_t buffsize, uint32_t steps, uint32_t p2p_chunk);

/* ---- R2: one request -> nqps pieces (plugin.cc:1467-1495) ------------------------------ */
/* chunk = DIVUP(DIVUP(size,nqps),128)*128; piece q: off = q*chunk, len = min(size-off, chunk);
 * len <= 0 is an empty work request (plugin.cc:1474-1476) reported as len 0.
 * Returns the piece stride (chunk).  off/len arrays hold nqps entries.  `int` arithmetic as in
 * the reference. */
int fl_qp_split(int size, int nqps, int* off, int* len);

/* ---- R3: live lane policy (fuselink.h:230-238) ----------------------------------------- */
int fl_lane_static(int channel_id, int n_nics);

/* ---- R4: refresh cadence (plugin.cc:38, 1443-1447, 1700-1712) -------------------------- */
/* receiver may switch lanes when n_finished % 8 == 0 and nothing received is unconsumed */
int fl_refresh_rx_due(int64_t n_finished, uint64_t received, uint64_t done);
/* sender refreshes its usage mask when (n_finished+1) % 8 == 0 */
int fl_refresh_tx_due(int64_t n_finished);

/* ---- R5: monitor state machine (monitor.h:40-55,191-250; monitor.cpp:159-193) ---------- */
typedef struct {
  int32_t tx_status[FLO_NGROUP][FLO_NNIC_PER_GROUP];
  int32_t rx_status[FLO_NGROUP][FLO_NNIC_PER_GROUP];
  int64_t tx_last_active[FLO_NGROUP][FLO_NNIC_PER_GROUP];
  int64_t rx_last_active[FLO_NGROUP][FLO_NNIC_PER_GROUP];
} fl_monitor_t;

void fl_mon_init(fl_monitor_t* m);
/* monitor.h:236-250: ts = now, status = BUSY */
void fl_mon_mark_tx(fl_monitor_t* m, int group, int nic, int64_t now);
void fl_mon_mark_rx(fl_monitor_t* m, int group, int nic, int64_t now);
/* monitor.cpp:159-193: keep status while ts + 160 > now, else IDLE */
void fl_mon_tick(fl_monitor_t* m, int64_t now);
/* monitor.h:191-206 as written: scans groups ascending, skips `group`, marks EVERY idle NIC
 * BORROWED (the break only leaves the inner loop) and returns the LAST one found, -1 if none. */
int  fl_mon_idle_pick_tx(fl_monitor_t* m, int group);
/* monitor.h:208-224: same with a NIC bitmask (bit i*NNIC_PER_GROUP+j) */
int  fl_mon_idle_pick_rx(fl_monitor_t* m, int group, int mask);
/* monitor.h:226-234: tx status of the first n NICs */
void fl_mon_status(const fl_monitor_t* m, int n_nics, int32_t* out);
/* Build-defined bridge from monitor state to integer credits: an IDLE lane gets `idle_credit`,
 * a BUSY or BORROWED lane gets 0, and the comm's own lane never drops below 1. */
void fl_credits_from_status(const int32_t* status, int n_lanes, int own_lane,
                            uint32_t idle_credit, uint32_t* credits);

/* Build-defined content of the sender's usage mask, which the reference leaves a placeholder (refreshTxUsage,
 * fuselink.h:261-267, always 0xffffffff; shipped as imm_data, plugin.cc:1441-1447, 1463; kept by the receiver as
 * txAvailable, plugin.cc:1884-1885): bit l set when lane l's send side is IDLE or l is the comm's own lane; bits from
 * n_lanes on are set. */
uint32_t fl_tx_usage_mask(const int32_t* tx_status, int n_lanes, int own_lane);
/* ... and what the receiver makes of it at its refresh (plugin.cc:1710; getIdleNicRx's mask, monitor.h:208-224): a lane
 * gets idle_credit when its receive side is IDLE and the mask admits it; the own lane never below 1.  With a mask of all
 * ones this is fl_credits_from_status over the receive statuses. */
void fl_rx_credits_from_status(const int32_t* rx_status, int n_lanes, int own_lane, uint32_t idle_credit,
                               uint32_t tx_mask, uint32_t* credits);

/* ---- R5 (build-defined): credit-weighted chunk -> lane schedule ------------------------- */
/*
 * Inputs: sizes s[0..n), L <= 16 lanes, credit rows c[r][0..L) (R rows), epoch length E chunks
 * (0 = one epoch), quantum q > 0, tile size T > 0, optional explicit source offsets, carry-in
 * state.  For chunk i with global index g = k0 + i:  epoch e = E ? g / E : 0, row r = e mod R,
 * W = sum_l c[r][l],  P_i = bytes of earlier chunks of the same epoch (carry-in included),
 * slot = floor(P_i / q) mod W,  lane_i = the l with K_l <= slot < K_l + c[r][l] (K = exclusive
 * prefix of the row).  A row with W == 0 (no lane has credit) is replaced by equal credits c = 1,
 * i.e. round-robin over the lanes as in the static policy (fuselink.h:235), and raises
 * FLO_SCHED_F_NO_CREDIT.  win_off_i = lane_off_in[lane_i] + bytes of
 * earlier chunks of this call on the same lane.  tile_base_i = sum_{j<i} ceil(s_j / T).
 * src_off_i = src_off[i] if given, else src_base + sum_{j<i} s_j.
 *
 * Properties that pin it: (1) equal credits and uniform chunks of q bytes -> lane_i = i mod L
 * (fuselink.h:235); (2) a lane with credit 0 receives nothing; (3) over W consecutive quanta of
 * one epoch lane l receives exactly c_l quanta; (4) sum of lane bytes == sum of sizes;
 * (5) integer-exact.
 */
typedef struct {
  uint64_t src_off;   /* byte offset of the chunk in the user buffer */
  uint64_t win_off;   /* byte offset inside the lane's staging window */
  uint32_t len;       /* bytes */
  uint32_t lane;      /* staging window / virtual NIC */
  uint32_t tile_base; /* exclusive prefix of ceil(len / tile) */
  uint32_t epoch;     /* credit epoch of the chunk (low 32 bits) */
} fl_chunk_desc_t;    /* 32 bytes; the device table uses the same layout */

typedef struct {
  uint64_t epoch_bytes;                 /* P carried into the next call */
  uint64_t chunk_index;                 /* k0 */
  uint64_t lane_off[FLO_MAX_NIC_NUM];   /* running in-window offsets */
} fl_sched_state_t;

typedef struct {
  uint64_t total_bytes;
  uint32_t total_tiles;
  uint32_t n_chunks;
  uint32_t flags;
  uint32_t uniform_tiles;                /* tiles per chunk when the split is uniform (sizes == NULL), else 0 */
  uint64_t lane_bytes[FLO_MAX_NIC_NUM];  /* bytes assigned to each lane by this call */
  uint32_t lane_chunks[FLO_MAX_NIC_NUM]; /* chunks assigned to each lane by this call */
} fl_sched_hdr_t;

#define FLO_SCHED_F_NO_CREDIT 1u
/* mode bits of the `mode` argument */
#define FLO_SCHED_RESET_OFFSETS 1u /* ignore state->lane_off on entry: windows are reused from 0 */
#define FLO_SCHED_NEW_EPOCH     4u /* ignore state->epoch_bytes on entry: a credit refresh starts a new epoch */
#define FLO_SCHED_MIRROR        2u /* win_off = src_off: the window mirrors the user buffer, which is
                                      the reference's translation window + (data - start_addr),
                                      plugin.cc:1582,1626 */

/* sizes == NULL means the uniform split of total_bytes by chunk_bytes (R1) */
int fl_credit_schedule(const uint32_t* sizes, uint64_t total_bytes, uint32_t chunk_bytes,
                       const uint64_t* src_off, uint64_t src_base, uint32_t n, uint32_t n_lanes,
                       const uint32_t* credits, uint32_t n_rows, uint32_t epoch_len,
                       uint64_t quantum, uint32_t tile_bytes, uint32_t mode, fl_sched_state_t* state,
                       fl_chunk_desc_t* table, fl_sched_hdr_t* hdr);

/* The same rows in destination order, for the striping side: grouped by lane, chunk order kept
 * inside a lane (so window offsets ascend), the lane of the last chunk placed last so that a short
 * final chunk stays the final row; tile_base = position * tiles_per_chunk.  Uniform splits only. */
int fl_table_by_lane(const fl_chunk_desc_t* table, uint32_t n, uint32_t n_lanes, uint32_t tiles_per_chunk,
                     fl_chunk_desc_t* out);

/* ---- R6: staging geometry and pointer translation --------------------------------------- */
/* fuselink.cc:29: aligned = ceil(size / gran) * gran (granularity queried BEFORE use; the
 * reference divides by a zero granularity first at fuselink.cc:15-18) */
uint64_t fl_align_up(uint64_t size, uint64_t gran);
/* number of 2 MiB units backing one window of `size` bytes (cumem.cu:145-147) */
uint64_t fl_window_units(uint64_t size, uint64_t unit);
/* plugin.cc:1582,1626: staged = window_base + (data - start_addr) */
uint64_t fl_translate(uint64_t window_base, uint64_t data, uint64_t start_addr);
/* plugin.cc:1201: relay GPU = (gpu_id + channelId) % NGPUs */
int      fl_relay_gpu(int gpu_id, int channel_id, int n_gpus);
/* plugin.cc:1181-1182: page-aligned base and page count of [data, data+size) */
void     fl_page_span(uint64_t data, uint64_t size, uint64_t page, uint64_t* addr, uint64_t* pages);

/* region cache + refcount (plugin.cc:1212-1227, 1326, 1337-1408): k registrations of the same
 * base share one region; the region dies on the k-th deregistration. */
typedef struct { uint64_t base[64]; int nrefs[64]; int n; int created; int destroyed; } fl_regcache_t;
void fl_regcache_init(fl_regcache_t* c);
int  fl_regcache_reg(fl_regcache_t* c, uint64_t base);   /* returns nrefs after the call */
int  fl_regcache_dereg(fl_regcache_t* c, uint64_t base); /* returns nrefs after, -1 unknown */

/* ---- R7: 2 MiB unit pool, first fit (cumem.cu:107-184) ---------------------------------- */
typedef struct { uint8_t mapped[FLO_MAX_MEM_TABLE_SIZE]; uint64_t va[FLO_MAX_MEM_TABLE_SIZE]; } fl_pool_t;
void fl_pool_init(fl_pool_t* p);
/* maps ceil(size/2MiB) consecutive 2 MiB steps starting at `base`, each onto the first unmapped
 * slot; writes slot ids to slots[]; returns steps mapped, or -1 when the pool runs out
 * (cumem.cu:176-179; slots mapped before the failure stay mapped, as in the reference). */
int  fl_pool_register(fl_pool_t* p, uint64_t base, uint64_t size, int* slots, int max_slots);
/* release the slot that backs `va` (cumem.cu:60-70, with the is_mapped flag actually cleared,
 * which the reference forgets); returns slot or -1 */
int  fl_pool_release(fl_pool_t* p, uint64_t va);
int  fl_pool_lookup(const fl_pool_t* p, uint64_t va); /* cumem.cu:186-193 */

/* ---- R8: request slots and FIFO handshake ----------------------------------------------- */
typedef struct { uint8_t used[FLO_MAX_REQUESTS]; } fl_reqtab_t;
void fl_reqtab_init(fl_reqtab_t* t);
int  fl_reqtab_get(fl_reqtab_t* t);         /* first free of 256, -1 if none (plugin.cc:1070-1085) */
void fl_reqtab_free(fl_reqtab_t* t, int i); /* plugin.cc:1086-1090 */
/* FIFO: receiver writes slot tail%256 with idx = tail+1 (plugin.cc:1619,1632); sender matches
 * slot head%256 only if its idx == head+1 (plugin.cc:1510-1514). */
typedef struct { uint64_t idx[FLO_MAX_REQUESTS]; uint64_t head, tail; } fl_fifo_t;
void fl_fifo_init(fl_fifo_t* f);
int  fl_fifo_post(fl_fifo_t* f);            /* returns slot */
int  fl_fifo_match(fl_fifo_t* f);           /* returns slot or -1 (would block) */

/* ---- CPU striping baseline (host memcpy) ------------------------------------------------ */
/* stripe: windows[lane] + win_off <- src + src_off ; reassemble is the inverse.
 * lo/hi select a chunk sub-range so callers can thread it. */
void fl_cpu_stripe(const uint8_t* src, uint8_t* const* windows, const fl_chunk_desc_t* table,
                   uint32_t lo, uint32_t hi);
void fl_cpu_reassemble(uint8_t* dst, const uint8_t* const* windows, const fl_chunk_desc_t* table,
                       uint32_t lo, uint32_t hi);
/* one thread per lane (threads = min(lanes, max_threads)), each handling its lane's chunks */
void fl_cpu_stripe_mt(const uint8_t* src, uint8_t* const* windows, const fl_chunk_desc_t* table,
                      uint32_t n, uint32_t n_lanes, int threads);
void fl_cpu_reassemble_mt(uint8_t* dst, const uint8_t* const* windows, const fl_chunk_desc_t* table,
                          uint32_t n, uint32_t n_lanes, int threads);
/* paged gather: chunk c of the table covers pages page_table[c*ppc .. (c+1)*ppc) of a pool whose
 * pages are page_bytes long; the receive side scatters them back to the same page numbers. */
void fl_cpu_gather_pages(const uint8_t* pool, const uint32_t* page_table, uint32_t page_bytes,
                         uint32_t pages_per_chunk, uint8_t* const* windows,
                         const fl_chunk_desc_t* table, uint32_t n);
void fl_cpu_scatter_pages(uint8_t* pool, const uint32_t* page_table, uint32_t page_bytes,
                          uint32_t pages_per_chunk, const uint8_t* const* windows,
                          const fl_chunk_desc_t* table, uint32_t n);
/* timed host-memcpy striping: runs stripe+reassemble `iters` times after `warm` warm-ups over
 * freshly allocated, pre-faulted 2 MiB-aligned lane windows, asserts memcmp(dst, src) == 0 each
 * run, returns the median seconds per stripe+reassemble (best in *best_s), <0 on mismatch. */
double fl_cpu_baseline_run(const uint8_t* src, uint64_t nbytes, const fl_chunk_desc_t* table,
                           const fl_sched_hdr_t* hdr, uint32_t n, uint32_t n_lanes, int threads,
                           int warm, int iters, double* best_s);
int fl_cpu_cores(void);

#ifdef __cplusplus
}
#endif
#endif /* FL_ORACLE_H_ */
