/*
 * fl_oracle.c -- CPU restatement of FuseLink's chunking / lane / staging arithmetic.
 * TEST INFRASTRUCTURE ONLY (see fl_oracle.h).  Plain C11, no HIP.
 */
#define _GNU_SOURCE
#include "fl_oracle.h"

#include <pthread.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>
#include <unistd.h>

/* ---- R1 ---------------------------------------------------------------------------------- */
uint64_t fl_split_count(uint64_t nbytes, uint32_t chunk) {
  if (chunk == 0) return 0;
  return (nbytes + chunk - 1) / chunk;
}

void fl_split_get(uint64_t nbytes, uint32_t chunk, uint64_t i, uint64_t* off, uint32_t* len) {
  uint64_t o = i * (uint64_t)chunk;
  uint64_t rem = o < nbytes ? nbytes - o : 0;
  *off = o;
  *len = (uint32_t)(rem < chunk ? rem : chunk);
}

uint32_t fl_step_size(uint64_t buffsize, uint32_t steps, uint32_t p2p_chunk) {
  /* stepSize = buffSize / NCCL_STEPS (fuselink.h:14); a net chunk never exceeds
   * NCCL_P2P_NET_CHUNKSIZE (run_bw_test.sbatch:34) */
  uint64_t step = buffsize / steps;
  return (uint32_t)(step < p2p_chunk ? step : p2p_chunk);
}

/* ---- R2 (plugin.cc:1467-1495) -------------------------------------------------------------- */
#define FLO_DIVUP(x, y) (((x) + (y)-1) / (y))
int fl_qp_split(int size, int nqps, int* off, int* len) {
  const int align = FLO_QP_ALIGN;                                  /* plugin.cc:1468 */
  int chunk = FLO_DIVUP(FLO_DIVUP(size, nqps), align) * align;     /* plugin.cc:1472 */
  int offset = 0;                                                  /* send.offset, plugin.cc:1585 */
  for (int q = 0; q < nqps; q++) {
    int length = size - offset < chunk ? size - offset : chunk;    /* plugin.cc:1473 */
    off[q] = offset;
    len[q] = length <= 0 ? 0 : length;                             /* plugin.cc:1474-1481 */
    offset += chunk;                                               /* plugin.cc:1491 */
  }
  return chunk;
}

/* ---- R3 (fuselink.h:235) --------------------------------------------------------------------- */
int fl_lane_static(int channel_id, int n_nics) { return channel_id % n_nics; }

/* ---- R4 ---------------------------------------------------------------------------------------- */
int fl_refresh_rx_due(int64_t n_finished, uint64_t received, uint64_t done) {
  if (n_finished % FLO_N_FINISHED_BATCH != 0) return 0;            /* plugin.cc:1700 */
  return received == done;                                         /* plugin.cc:1704-1709 */
}
int fl_refresh_tx_due(int64_t n_finished) {
  return (n_finished + 1) % FLO_N_FINISHED_BATCH == 0;             /* plugin.cc:1443 */
}

/* ---- R5: monitor --------------------------------------------------------------------------- */
void fl_mon_init(fl_monitor_t* m) { memset(m, 0, sizeof(*m)); }

void fl_mon_mark_tx(fl_monitor_t* m, int group, int nic, int64_t now) {
  m->tx_last_active[group][nic] = now;                             /* monitor.h:238 */
  m->tx_status[group][nic] = FLO_NIC_BUSY;                         /* monitor.h:240 */
}
void fl_mon_mark_rx(fl_monitor_t* m, int group, int nic, int64_t now) {
  m->rx_last_active[group][nic] = now;                             /* monitor.h:246 */
  m->rx_status[group][nic] = FLO_NIC_BUSY;                         /* monitor.h:248 */
}

void fl_mon_tick(fl_monitor_t* m, int64_t now) {
  for (int i = 0; i < FLO_NGROUP; ++i) {
    for (int j = 0; j < FLO_NNIC_PER_GROUP; ++j) {
      if (m->tx_last_active[i][j] + FLO_MONITOR_TIMEOUT_US > now) { /* monitor.cpp:172 keep */
      } else {
        m->tx_status[i][j] = FLO_NIC_IDLE;                          /* monitor.cpp:176 */
      }
    }
    for (int j = 0; j < FLO_NNIC_PER_GROUP; ++j) {
      if (m->rx_last_active[i][j] + FLO_MONITOR_TIMEOUT_US > now) { /* monitor.cpp:181 keep */
      } else {
        m->rx_status[i][j] = FLO_NIC_IDLE;                          /* monitor.cpp:185 */
      }
    }
  }
}

int fl_mon_idle_pick_tx(fl_monitor_t* m, int group) {
  int idle = -1;
  for (int i = 0; i < FLO_NGROUP; ++i) {
    if (i == group) continue;                                       /* monitor.h:195 */
    for (int j = 0; j < FLO_NNIC_PER_GROUP; ++j) {
      if (m->tx_status[i][j] == FLO_NIC_IDLE) {                     /* monitor.h:197 */
        idle = i * FLO_NNIC_PER_GROUP + j;
        m->tx_status[i][j] = FLO_NIC_BORROWED;                      /* monitor.h:199 */
        break; /* leaves the inner loop only (monitor.h:200) */
      }
    }
  }
  return idle;
}

int fl_mon_idle_pick_rx(fl_monitor_t* m, int group, int mask) {
  int idle = -1;
  for (int i = 0; i < FLO_NGROUP; ++i) {
    if (i == group) continue;                                       /* monitor.h:212 */
    for (int j = 0; j < FLO_NNIC_PER_GROUP; ++j) {
      if ((mask & (1 << (i * FLO_NNIC_PER_GROUP + j))) == 0) continue; /* monitor.h:214 */
      if (m->rx_status[i][j] == FLO_NIC_IDLE) {
        idle = i * FLO_NNIC_PER_GROUP + j;
        m->rx_status[i][j] = FLO_NIC_BORROWED;
        break;
      }
    }
  }
  return idle;
}

void fl_mon_status(const fl_monitor_t* m, int n_nics, int32_t* out) {
  for (int i = 0; i < n_nics; ++i) {
    int p = i / FLO_NNIC_PER_GROUP, q = i % FLO_NNIC_PER_GROUP;     /* monitor.h:229-230 */
    out[i] = m->tx_status[p][q];
  }
}

void fl_credits_from_status(const int32_t* status, int n_lanes, int own_lane,
                            uint32_t idle_credit, uint32_t* credits) {
  for (int l = 0; l < n_lanes; ++l) credits[l] = status[l] == FLO_NIC_IDLE ? idle_credit : 0;
  if (own_lane >= 0 && own_lane < n_lanes && credits[own_lane] == 0) credits[own_lane] = 1;
}

/* refreshTxUsage (fuselink.h:265-267) is a placeholder that returns 0xffffffff; the mask it stands for is read off the
 * sender's statuses: bit l set when lane l's send side is IDLE, the comm's own lane always, and every bit from n_lanes
 * on (so that a table in which nothing is busy gives the placeholder's value). */
uint32_t fl_tx_usage_mask(const int32_t* tx_status, int n_lanes, int own_lane) {
  uint32_t mask = n_lanes >= 32 ? 0u : ~0u << n_lanes;
  for (int l = 0; l < n_lanes && l < 32; ++l)
    if (tx_status[l] == FLO_NIC_IDLE || l == own_lane) mask |= 1u << l;
  return mask;
}

/* The receiver's side of the same decision: getIdleNicRx(group, priority, txAvailable) skips every NIC that the mask does
 * not admit (monitor.h:214, the call commented out at fuselink.h:240-243); as credits, a lane counts when its receive side
 * is IDLE and the sender's mask admits it; the own lane never drops below 1. */
void fl_rx_credits_from_status(const int32_t* rx_status, int n_lanes, int own_lane, uint32_t idle_credit,
                               uint32_t tx_mask, uint32_t* credits) {
  for (int l = 0; l < n_lanes; ++l)
    credits[l] = rx_status[l] == FLO_NIC_IDLE && (l >= 32 || ((tx_mask >> l) & 1u)) ? idle_credit : 0;
  if (own_lane >= 0 && own_lane < n_lanes && credits[own_lane] == 0) credits[own_lane] = 1;
}

/* ---- R5: build-defined credit schedule ------------------------------------------------------ */
int fl_credit_schedule(const uint32_t* sizes, uint64_t total_bytes, uint32_t chunk_bytes,
                       const uint64_t* src_off, uint64_t src_base, uint32_t n, uint32_t n_lanes,
                       const uint32_t* credits, uint32_t n_rows, uint32_t epoch_len,
                       uint64_t quantum, uint32_t tile_bytes, uint32_t mode, fl_sched_state_t* state,
                       fl_chunk_desc_t* table, fl_sched_hdr_t* hdr) {
  if (n_lanes == 0 || n_lanes > FLO_MAX_NIC_NUM || n_rows == 0 || quantum == 0 || tile_bytes == 0)
    return -1;
  if (!sizes && n && chunk_bytes == 0) return -1;
  fl_sched_state_t st;
  if (state) st = *state; else memset(&st, 0, sizeof(st));
  fl_sched_hdr_t h;
  memset(&h, 0, sizeof(h));
  uint64_t P = (mode & FLO_SCHED_NEW_EPOCH) ? 0 : st.epoch_bytes;
  uint64_t run = 0;
  uint64_t lane_off[FLO_MAX_NIC_NUM];
  for (int l = 0; l < FLO_MAX_NIC_NUM; ++l) lane_off[l] = (mode & FLO_SCHED_RESET_OFFSETS) ? 0 : st.lane_off[l];
  uint32_t tiles = 0;
  for (uint32_t i = 0; i < n; ++i) {
    uint64_t g = st.chunk_index + i;
    uint64_t e = epoch_len ? g / epoch_len : 0;
    if (epoch_len && g % epoch_len == 0) P = 0; /* P restarts at an epoch boundary */
    uint32_t s;
    if (sizes) s = sizes[i];
    else { uint64_t o; fl_split_get(total_bytes, chunk_bytes, i, &o, &s); }
    const uint32_t* row = credits + (size_t)(e % n_rows) * n_lanes;
    uint64_t W = 0;
    for (uint32_t l = 0; l < n_lanes; ++l) W += row[l];
    uint32_t ones[FLO_MAX_NIC_NUM];
    if (W == 0) {                                 /* every lane busy: equal credits stand in, which */
      for (uint32_t l = 0; l < n_lanes; ++l) ones[l] = 1; /* is the round-robin of fuselink.h:235 */
      row = ones;
      W = n_lanes;
      h.flags |= FLO_SCHED_F_NO_CREDIT;
    }
    uint32_t lane = 0;
    {
      uint64_t slot = (P / quantum) % W;
      uint64_t K = 0;
      for (uint32_t l = 0; l < n_lanes; ++l) {
        if (slot >= K && slot < K + row[l]) { lane = l; break; }
        K += row[l];
      }
    }
    table[i].src_off = src_off ? src_off[i] : src_base + run;
    table[i].win_off = (mode & FLO_SCHED_MIRROR) ? table[i].src_off : lane_off[lane];
    table[i].len = s;
    table[i].lane = lane;
    table[i].tile_base = tiles;
    table[i].epoch = (uint32_t)e;
    lane_off[lane] += s;
    h.lane_bytes[lane] += s;
    h.lane_chunks[lane] += 1;
    tiles += (s + tile_bytes - 1) / tile_bytes;
    P += s;
    run += s;
  }
  h.total_bytes = run;
  h.total_tiles = tiles;
  h.n_chunks = n;
  h.uniform_tiles = (!sizes && n) ? (chunk_bytes + tile_bytes - 1) / tile_bytes : 0;
  if (hdr) *hdr = h;
  if (state) {
    state->epoch_bytes = P;
    state->chunk_index = st.chunk_index + n;
    for (int l = 0; l < FLO_MAX_NIC_NUM; ++l) state->lane_off[l] = lane_off[l];
  }
  return 0;
}

int fl_table_by_lane(const fl_chunk_desc_t* table, uint32_t n, uint32_t n_lanes, uint32_t tiles_per_chunk,
                     fl_chunk_desc_t* out) {
  if (n_lanes == 0 || n_lanes > FLO_MAX_NIC_NUM || (n && (!table || !out))) return -1;
  if (n == 0) return 0;
  uint64_t count[FLO_MAX_NIC_NUM] = {0}, base[FLO_MAX_NIC_NUM] = {0};
  for (uint32_t i = 0; i < n; ++i) {
    if (table[i].lane >= n_lanes) return -1;
    count[table[i].lane]++;
  }
  const uint32_t lane_last = table[n - 1].lane;
  uint64_t run = 0;
  for (uint32_t k = 0; k < n_lanes; ++k) {
    const uint32_t l = (lane_last + 1 + k) % n_lanes;
    base[l] = run;
    run += count[l];
  }
  for (uint32_t i = 0; i < n; ++i) {
    const uint64_t pos = base[table[i].lane]++;
    out[pos] = table[i];
    out[pos].tile_base = (uint32_t)(pos * tiles_per_chunk);
  }
  return 0;
}

/* ---- R6 ------------------------------------------------------------------------------------- */
uint64_t fl_align_up(uint64_t size, uint64_t gran) { return ((size + gran - 1) / gran) * gran; } /* fuselink.cc:29 */
uint64_t fl_window_units(uint64_t size, uint64_t unit) { return (size + unit - 1) / unit; }      /* cumem.cu:146-147 */
uint64_t fl_translate(uint64_t window_base, uint64_t data, uint64_t start_addr) {
  return window_base + data - start_addr;                                                         /* plugin.cc:1582 */
}
int fl_relay_gpu(int gpu_id, int channel_id, int n_gpus) { return (gpu_id + channel_id) % n_gpus; } /* plugin.cc:1201 */
void fl_page_span(uint64_t data, uint64_t size, uint64_t page, uint64_t* addr, uint64_t* pages) {
  uint64_t a = data & ~(page - 1);                                                                /* plugin.cc:1181 */
  *addr = a;
  *pages = (data + size - a + page - 1) / page;                                                   /* plugin.cc:1182 */
}

void fl_regcache_init(fl_regcache_t* c) { memset(c, 0, sizeof(*c)); }
int fl_regcache_reg(fl_regcache_t* c, uint64_t base) {
  for (int i = 0; i < c->n; ++i)
    if (c->base[i] == base) return ++c->nrefs[i];                   /* plugin.cc:1214-1226 */
  if (c->n == 64) return -1;
  c->base[c->n] = base;
  c->nrefs[c->n] = 1;                                               /* plugin.cc:1241 */
  c->n++;
  c->created++;
  return 1;
}
int fl_regcache_dereg(fl_regcache_t* c, uint64_t base) {
  for (int i = 0; i < c->n; ++i) {
    if (c->base[i] != base) continue;
    int r = --c->nrefs[i];                                          /* plugin.cc:1347 */
    if (r == 0) {                                                   /* plugin.cc:1382-1403 */
      c->base[i] = c->base[c->n - 1];
      c->nrefs[i] = c->nrefs[c->n - 1];
      c->n--;
      c->destroyed++;
    }
    return r;
  }
  return -1;
}

/* ---- R7 ------------------------------------------------------------------------------------- */
void fl_pool_init(fl_pool_t* p) { memset(p, 0, sizeof(*p)); }

int fl_pool_register(fl_pool_t* p, uint64_t base, uint64_t size, int* slots, int max_slots) {
  uint64_t steps = (size + FLO_BUFFER_UNIT - 1) / FLO_BUFFER_UNIT;  /* cumem.cu:146-147 (64-bit) */
  uint64_t va = base;
  for (uint64_t i = 0; i < steps; ++i) {
    int found = -1;
    for (int j = 0; j < FLO_MAX_MEM_TABLE_SIZE; ++j) {              /* cumem.cu:157 */
      if (!p->mapped[j]) { found = j; break; }                      /* cumem.cu:158 first fit */
    }
    if (found < 0) return -1;                                       /* cumem.cu:176-179 */
    p->mapped[found] = 1;                                           /* cumem.cu:164 */
    p->va[found] = va;                                              /* cumem.cu:165 */
    if ((int)i < max_slots && slots) slots[i] = found;
    va += FLO_BUFFER_UNIT;                                          /* cumem.cu:181 */
  }
  return (int)steps;
}

int fl_pool_lookup(const fl_pool_t* p, uint64_t va) {
  for (int j = 0; j < FLO_MAX_MEM_TABLE_SIZE; ++j)
    if (p->mapped[j] && p->va[j] == va) return j;
  return -1;
}

int fl_pool_release(fl_pool_t* p, uint64_t va) {
  int j = fl_pool_lookup(p, va);
  if (j < 0) return -1;                                             /* cumem.cu:62-65 */
  p->mapped[j] = 0;
  p->va[j] = 0;
  return j;
}

/* ---- R8 ------------------------------------------------------------------------------------- */
void fl_reqtab_init(fl_reqtab_t* t) { memset(t, 0, sizeof(*t)); }
int fl_reqtab_get(fl_reqtab_t* t) {
  for (int i = 0; i < FLO_MAX_REQUESTS; ++i)
    if (!t->used[i]) { t->used[i] = 1; return i; }                  /* plugin.cc:1071-1080 */
  return -1;                                                        /* plugin.cc:1082-1084 */
}
void fl_reqtab_free(fl_reqtab_t* t, int i) { t->used[i] = 0; }      /* plugin.cc:1087 */

void fl_fifo_init(fl_fifo_t* f) { memset(f, 0, sizeof(*f)); }
int fl_fifo_post(fl_fifo_t* f) {
  int slot = (int)(f->tail % FLO_MAX_REQUESTS);                     /* plugin.cc:1619 */
  f->idx[slot] = f->tail + 1;                                       /* plugin.cc:1632 */
  f->tail++;                                                        /* plugin.cc:1675 */
  return slot;
}
int fl_fifo_match(fl_fifo_t* f) {
  int slot = (int)(f->head % FLO_MAX_REQUESTS);                     /* plugin.cc:1510 */
  if (f->idx[slot] != f->head + 1) return -1;                       /* plugin.cc:1513-1514 */
  f->idx[slot] = 0;                                                 /* plugin.cc:1605 */
  f->head++;                                                        /* plugin.cc:1607 */
  return slot;
}

/* ---- CPU striping baseline ------------------------------------------------------------------ */
void fl_cpu_stripe(const uint8_t* src, uint8_t* const* windows, const fl_chunk_desc_t* table,
                   uint32_t lo, uint32_t hi) {
  for (uint32_t i = lo; i < hi; ++i)
    memcpy(windows[table[i].lane] + table[i].win_off, src + table[i].src_off, table[i].len);
}

void fl_cpu_reassemble(uint8_t* dst, const uint8_t* const* windows, const fl_chunk_desc_t* table,
                       uint32_t lo, uint32_t hi) {
  for (uint32_t i = lo; i < hi; ++i)
    memcpy(dst + table[i].src_off, windows[table[i].lane] + table[i].win_off, table[i].len);
}

typedef struct {
  int dir, tid, threads;
  const uint8_t* src;
  uint8_t* dst;
  uint8_t* const* windows;
  const fl_chunk_desc_t* table;
  uint32_t n, n_lanes;
} fl_mt_job_t;

static void* fl_mt_worker(void* arg) {
  fl_mt_job_t* j = (fl_mt_job_t*)arg;
#ifdef __linux__
  cpu_set_t set;
  CPU_ZERO(&set);
  long ncpu = sysconf(_SC_NPROCESSORS_ONLN);
  if (ncpu > 0) { CPU_SET(j->tid % ncpu, &set); pthread_setaffinity_np(pthread_self(), sizeof(set), &set); }
#endif
  for (uint32_t i = 0; i < j->n; ++i) {
    const fl_chunk_desc_t* d = &j->table[i];
    if ((int)(d->lane % (uint32_t)j->threads) != j->tid) continue; /* one thread per lane */
    if (j->dir == 0) memcpy(j->windows[d->lane] + d->win_off, j->src + d->src_off, d->len);
    else memcpy(j->dst + d->src_off, j->windows[d->lane] + d->win_off, d->len);
  }
  return NULL;
}

static void fl_mt_run(int dir, const uint8_t* src, uint8_t* dst, uint8_t* const* windows,
                      const fl_chunk_desc_t* table, uint32_t n, uint32_t n_lanes, int threads) {
  if (threads < 1) threads = 1;
  if ((uint32_t)threads > n_lanes) threads = (int)n_lanes;
  pthread_t th[FLO_MAX_NIC_NUM];
  fl_mt_job_t jobs[FLO_MAX_NIC_NUM];
  for (int t = 0; t < threads; ++t) {
    jobs[t] = (fl_mt_job_t){dir, t, threads, src, dst, windows, table, n, n_lanes};
    pthread_create(&th[t], NULL, fl_mt_worker, &jobs[t]);
  }
  for (int t = 0; t < threads; ++t) pthread_join(th[t], NULL);
}

void fl_cpu_stripe_mt(const uint8_t* src, uint8_t* const* windows, const fl_chunk_desc_t* table,
                      uint32_t n, uint32_t n_lanes, int threads) {
  fl_mt_run(0, src, NULL, windows, table, n, n_lanes, threads);
}
void fl_cpu_reassemble_mt(uint8_t* dst, const uint8_t* const* windows, const fl_chunk_desc_t* table,
                          uint32_t n, uint32_t n_lanes, int threads) {
  fl_mt_run(1, NULL, dst, (uint8_t* const*)windows, table, n, n_lanes, threads);
}

void fl_cpu_gather_pages(const uint8_t* pool, const uint32_t* page_table, uint32_t page_bytes,
                         uint32_t pages_per_chunk, uint8_t* const* windows,
                         const fl_chunk_desc_t* table, uint32_t n) {
  for (uint32_t c = 0; c < n; ++c) {
    uint32_t np = (table[c].len + page_bytes - 1) / page_bytes;
    for (uint32_t k = 0; k < np; ++k) {
      uint32_t pg = page_table[(size_t)c * pages_per_chunk + k];
      uint32_t len = table[c].len - k * page_bytes < page_bytes ? table[c].len - k * page_bytes : page_bytes;
      memcpy(windows[table[c].lane] + table[c].win_off + (size_t)k * page_bytes,
             pool + (size_t)pg * page_bytes, len);
    }
  }
}

void fl_cpu_scatter_pages(uint8_t* pool, const uint32_t* page_table, uint32_t page_bytes,
                          uint32_t pages_per_chunk, const uint8_t* const* windows,
                          const fl_chunk_desc_t* table, uint32_t n) {
  for (uint32_t c = 0; c < n; ++c) {
    uint32_t np = (table[c].len + page_bytes - 1) / page_bytes;
    for (uint32_t k = 0; k < np; ++k) {
      uint32_t pg = page_table[(size_t)c * pages_per_chunk + k];
      uint32_t len = table[c].len - k * page_bytes < page_bytes ? table[c].len - k * page_bytes : page_bytes;
      memcpy(pool + (size_t)pg * page_bytes,
             windows[table[c].lane] + table[c].win_off + (size_t)k * page_bytes, len);
    }
  }
}

int fl_cpu_cores(void) {
  long n = sysconf(_SC_NPROCESSORS_ONLN);
  return n > 0 ? (int)n : 1;
}

static double fl_now_s(void) {
  struct timespec ts;
  clock_gettime(CLOCK_MONOTONIC, &ts); /* as clockNano, src/extern/utils.h:47-51 */
  return (double)ts.tv_sec + 1e-9 * (double)ts.tv_nsec;
}

static int fl_cmp_double(const void* a, const void* b) {
  double x = *(const double*)a, y = *(const double*)b;
  return x < y ? -1 : x > y;
}

double fl_cpu_baseline_run(const uint8_t* src, uint64_t nbytes, const fl_chunk_desc_t* table,
                           const fl_sched_hdr_t* hdr, uint32_t n, uint32_t n_lanes, int threads,
                           int warm, int iters, double* best_s) {
  uint8_t* windows[FLO_MAX_NIC_NUM] = {0};
  for (uint32_t l = 0; l < n_lanes; ++l) {
    uint64_t cap = fl_align_up(hdr->lane_bytes[l] ? hdr->lane_bytes[l] : 1, FLO_BUFFER_UNIT);
    windows[l] = (uint8_t*)aligned_alloc(FLO_BUFFER_UNIT, cap);
    if (!windows[l]) return -2.0;
    memset(windows[l], 0, cap); /* pre-fault */
  }
  uint8_t* dst = (uint8_t*)aligned_alloc(FLO_BUFFER_UNIT, fl_align_up(nbytes ? nbytes : 1, FLO_BUFFER_UNIT));
  if (!dst) return -2.0;
  memset(dst, 0, nbytes);
  if (iters < 1) iters = 1;
  double* t = (double*)malloc(sizeof(double) * (size_t)iters);
  double ret = 0.0;
  for (int it = -warm; it < iters; ++it) {
    double t0 = fl_now_s();
    if (threads <= 1) {
      fl_cpu_stripe(src, windows, table, 0, n);
      fl_cpu_reassemble(dst, (const uint8_t* const*)windows, table, 0, n);
    } else {
      fl_cpu_stripe_mt(src, windows, table, n, n_lanes, threads);
      fl_cpu_reassemble_mt(dst, (const uint8_t* const*)windows, table, n, n_lanes, threads);
    }
    double t1 = fl_now_s();
    if (memcmp(dst, src, nbytes) != 0) { ret = -1.0; break; }
    if (it >= 0) t[it] = t1 - t0;
  }
  if (ret == 0.0) {
    qsort(t, (size_t)iters, sizeof(double), fl_cmp_double);
    ret = t[iters / 2];
    if (best_s) *best_s = t[0];
  }
  free(t);
  free(dst);
  for (uint32_t l = 0; l < n_lanes; ++l) free(windows[l]);
  return ret;
}
