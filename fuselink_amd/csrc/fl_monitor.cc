// fl_monitor.cc -- lane (virtual NIC) idleness tracking and the credits derived from it.
//
// The reference keeps this state in POSIX shared memory owned by a daemon (FuseLink
// src/monitor.h:47-55, src/monitor.cpp:159-193) and guards every access with a named semaphore.
// The table here has the same layout and can live in two places:
//   * in the plugin's process behind a mutex (the default), with the clock passed in, so that the
//     state machine is deterministic;
//   * in the reference's shared-memory object (`/rdma_monitor_shm`, guarded by the named semaphore
//     `/rdma_monitor_sem`), after fl_monitor_attach_shm(): then several processes -- this library,
//     the fuselink-monitor daemon, the reference's own MonitorClient -- see one table.
// The transport marks a lane active when it puts traffic on it, a tick ages lanes to IDLE after
// MONITOR_TIMEOUT_US, and the scheduler's credits are read off the statuses at each refresh.
#include <fcntl.h>
#include <semaphore.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <atomic>
#include <cerrno>
#include <chrono>
#include <ctime>
#include <cstring>
#include <mutex>
#include <shared_mutex>

#include "fl_internal.h"
#include "fuselink_hip.h"
#include "fuselink_net.h"

namespace {

constexpr int kGroups = FL_NET_MAX_LANES;  // NGROUP with NNIC_PER_GROUP == 1 (src/monitor.h:18-20)
enum : int32_t { kIdle = 0, kBusy = 1, kBorrowed = 2 };  // NicStatus, src/monitor.h:40-44

// struct SharedMemory of src/monitor.h:47-55 with NGROUP = 16, NNIC_PER_GROUP = 1: two status arrays,
// two timestamp arrays (microseconds of the steady clock), the daemon's running flag.
struct LaneTable {
  int32_t tx_status[kGroups];
  int32_t rx_status[kGroups];
  int64_t tx_last_active[kGroups];
  int64_t rx_last_active[kGroups];
  volatile uint8_t running;
};
static_assert(offsetof(LaneTable, rx_status) == 64 && offsetof(LaneTable, tx_last_active) == 128 &&
              offsetof(LaneTable, rx_last_active) == 256 && offsetof(LaneTable, running) == 384 && sizeof(LaneTable) == 392,
              "layout must match the reference's SharedMemory");

// g_mu guards the pointers below against attach / detach (taken exclusively there).  A table access takes it
// exclusively in process-local mode, where it is the table's lock, and shared in shared-memory mode, where the
// cross-process semaphore is: a thread that waits for the semaphore then holds up nobody in this process.
std::shared_mutex g_mu;
LaneTable g_local = {};
LaneTable* g_tab = &g_local;
sem_t* g_sem = SEM_FAILED;  // the cross-process lock when attached
int g_shm_fd = -1;
bool g_owner = false;
char g_shm_name[64] = "", g_sem_name[64] = "";
std::atomic<bool> g_attached{false};   // g_sem != SEM_FAILED, readable without the lock
std::atomic<bool> g_manual_clock{false};
std::atomic<int64_t> g_manual_now{0};
// Set when a wait for the semaphore ran into its bound: a process died holding it.  From then on an access only tries
// the semaphore (and clears the flag when it gets it) instead of waiting again.
std::atomic<bool> g_sem_dead{false};

// Every access to the table goes through one of these.  The cross-process semaphore is waited for with a
// bound: a process that died holding it (the reference's sem_wait would then block for ever, src/monitor.h:195)
// must not stall a transport thread, so after kSemWaitMs the access goes ahead unlocked -- entries are single
// words, the worst outcome is one stale status -- and the semaphore is not posted.  Only the first such access pays
// the wait; the later ones try the semaphore without waiting until it is free again.
constexpr long kSemWaitMs = 200;
struct TableLock {
  std::unique_lock<std::shared_mutex> local;
  std::shared_lock<std::shared_mutex> shared;
  sem_t* sem = SEM_FAILED;
  bool held = false;
  TableLock() {
    if (!g_attached.load(std::memory_order_acquire)) {   // process-local table: g_mu is its lock
      local = std::unique_lock<std::shared_mutex>(g_mu);
      if (g_sem == SEM_FAILED) return;
      local.unlock();                   // attached meanwhile
    }
    shared = std::shared_lock<std::shared_mutex>(g_mu);
    if (g_sem == SEM_FAILED) return;    // detached meanwhile: one unlocked access to single words
    sem = g_sem;
    if (g_sem_dead.load(std::memory_order_acquire)) {
      held = sem_trywait(sem) == 0;
      if (held) g_sem_dead.store(false, std::memory_order_release);
      return;
    }
    timespec until;
    clock_gettime(CLOCK_REALTIME, &until);
    until.tv_nsec += kSemWaitMs * 1000000L;
    until.tv_sec += until.tv_nsec / 1000000000L;
    until.tv_nsec %= 1000000000L;
    int rc;
    while ((rc = sem_timedwait(sem, &until)) != 0 && errno == EINTR) {}
    held = rc == 0;
    if (!held) g_sem_dead.store(true, std::memory_order_release);
  }
  ~TableLock() {
    if (held) sem_post(sem);
  }
};

int32_t* status_of(int is_tx) { return is_tx ? g_tab->tx_status : g_tab->rx_status; }
int64_t* stamp_of(int is_tx) { return is_tx ? g_tab->tx_last_active : g_tab->rx_last_active; }

void detach_locked() {
  if (g_tab != &g_local) munmap(g_tab, sizeof(LaneTable));
  g_tab = &g_local;
  if (g_shm_fd >= 0) close(g_shm_fd);
  g_shm_fd = -1;
  if (g_sem != SEM_FAILED) sem_close(g_sem);
  g_sem = SEM_FAILED;
  g_attached.store(false, std::memory_order_release);
  if (g_owner) {
    shm_unlink(g_shm_name);
    sem_unlink(g_sem_name);
  }
  g_owner = false;
}

}  // namespace

extern "C" {

int fl_monitor_attach_shm(const char* shm_name, const char* sem_name, int create) {
  if (!shm_name) shm_name = "/rdma_monitor_shm";  // SHM_NAME, src/monitor.h:23
  if (!sem_name) sem_name = "/rdma_monitor_sem";  // SEM_NAME, src/monitor.h:24
  if (strlen(shm_name) >= sizeof(g_shm_name) || strlen(sem_name) >= sizeof(g_sem_name)) return fl_set_error(FLH_E_ARG, "name too long");
  std::unique_lock<std::shared_mutex> g(g_mu);
  g_sem_dead.store(false, std::memory_order_release);
  detach_locked();
  if (create) {  // the daemon's part (Monitor::setupSharedMemory in src/monitor.cpp)
    shm_unlink(shm_name);
    sem_unlink(sem_name);
  }
  int fd = shm_open(shm_name, create ? (O_CREAT | O_RDWR) : O_RDWR, 0666);
  if (fd < 0) return fl_set_error(FLH_E_STATE, "shm_open(%s) failed: is the monitor daemon running?", shm_name);
  if (create && ftruncate(fd, sizeof(LaneTable)) != 0) { close(fd); return fl_set_error(FLH_E_STATE, "ftruncate failed"); }
  struct stat st;
  if (fstat(fd, &st) != 0 || (size_t)st.st_size < sizeof(LaneTable)) { close(fd); return fl_set_error(FLH_E_STATE, "%s is smaller than the monitor table", shm_name); }
  void* p = mmap(nullptr, sizeof(LaneTable), PROT_READ | PROT_WRITE, MAP_SHARED, fd, 0);
  if (p == MAP_FAILED) { close(fd); return fl_set_error(FLH_E_STATE, "mmap of %s failed", shm_name); }
  sem_t* sem = create ? sem_open(sem_name, O_CREAT, 0666, 1) : sem_open(sem_name, 0);
  if (sem == SEM_FAILED) { munmap(p, sizeof(LaneTable)); close(fd); return fl_set_error(FLH_E_STATE, "sem_open(%s) failed", sem_name); }
  g_tab = (LaneTable*)p;
  g_shm_fd = fd;
  g_sem = sem;
  g_attached.store(true, std::memory_order_release);
  g_owner = create != 0;
  strcpy(g_shm_name, shm_name);
  strcpy(g_sem_name, sem_name);
  if (create) {
    memset(g_tab, 0, sizeof(LaneTable));
    g_tab->running = 1;
  }
  return FLH_OK;
}

int fl_monitor_detach(void) {
  std::unique_lock<std::shared_mutex> g(g_mu);
  if (g_owner && g_tab != &g_local) g_tab->running = 0;
  detach_locked();
  return FLH_OK;
}

int fl_monitor_is_shared(void) {
  std::shared_lock<std::shared_mutex> g(g_mu);
  return g_tab != &g_local;
}

int fl_monitor_daemon_running(void) {
  TableLock l;
  return g_tab != &g_local && g_tab->running != 0;
}

int fl_monitor_set_clock(int manual, int64_t now_us) {
  g_manual_now.store(now_us, std::memory_order_relaxed);
  g_manual_clock.store(manual != 0, std::memory_order_release);
  return FLH_OK;
}

// get_timestamp() of src/monitor.h:29-33 unless a test has frozen the clock
int64_t fl_monitor_now(void) {
  if (g_manual_clock.load(std::memory_order_acquire)) return g_manual_now.load(std::memory_order_relaxed);   // no lock on the request path
  return std::chrono::duration_cast<std::chrono::microseconds>(std::chrono::steady_clock::now().time_since_epoch()).count();
}

int fl_monitor_reset(void) {
  TableLock l;
  const uint8_t running = g_tab->running;
  memset(g_tab, 0, sizeof(LaneTable));
  g_tab->running = running;
  return FLH_OK;
}

// markNicTxAsActive / markNicRxAsActive (src/monitor.h:236-250)
int fl_monitor_mark_active(int lane, int is_tx, int64_t now_us) {
  if (lane < 0 || lane >= kGroups) return fl_set_error(FLH_E_ARG, "lane %d out of range", lane);
  TableLock l;
  stamp_of(is_tx)[lane] = now_us;
  status_of(is_tx)[lane] = kBusy;
  return FLH_OK;
}

int fl_monitor_set_entry(int lane, int is_tx, int32_t status, int64_t last_active_us) {
  if (lane < 0 || lane >= kGroups || status < kIdle || status > kBorrowed) return fl_set_error(FLH_E_ARG, "bad table entry");
  TableLock l;
  status_of(is_tx)[lane] = status;
  stamp_of(is_tx)[lane] = last_active_us;
  return FLH_OK;
}

// Monitor::monitorThread body (src/monitor.cpp:164-188): a lane whose last activity is at least the
// timeout old becomes IDLE, whatever it was (BUSY or BORROWED); a younger one keeps its status.
int fl_monitor_tick(int64_t now_us) {
  TableLock l;
  for (int d = 0; d < 2; ++d)
    for (int i = 0; i < kGroups; ++i)
      if (!(stamp_of(d)[i] + FL_NET_MONITOR_TIMEOUT_US > now_us)) status_of(d)[i] = kIdle;
  return FLH_OK;
}

// getNICStatus (src/monitor.h:226-234), for either direction
int fl_monitor_status(int is_tx, int n_lanes, int32_t* status_out) {
  if (n_lanes < 0 || n_lanes > kGroups || !status_out) return fl_set_error(FLH_E_ARG, "bad status query");
  TableLock l;
  for (int i = 0; i < n_lanes; ++i) status_out[i] = status_of(is_tx)[i];
  return FLH_OK;
}

// getIdleNicTx / getIdleNicRx (src/monitor.h:191-224).  As written there, the `break` leaves only
// the one-iteration inner loop, so the scan goes on: every idle NIC outside `group` that the mask
// admits is marked BORROWED and the last of them is returned.  exact != 0 stops at the first.
int fl_monitor_idle_pick(int is_tx, int group, int mask, int exact) {
  TableLock l;
  int32_t* st = status_of(is_tx);
  int found = -1;
  for (int i = 0; i < kGroups; ++i) {
    if (i == group) continue;
    if (!is_tx && (mask & (1 << i)) == 0) continue;  // only the rx query takes a mask (src/monitor.h:214)
    if (st[i] != kIdle) continue;
    st[i] = kBorrowed;
    found = i;
    if (exact) break;
  }
  return found;
}

// Give a borrowed lane back before its timeout runs out (the reference never does: a BORROWED NIC only
// returns to IDLE through the daemon's ageing, src/monitor.cpp:171-186).  Only a BORROWED entry changes.
int fl_monitor_release(int lane, int is_tx) {
  if (lane < 0 || lane >= kGroups) return fl_set_error(FLH_E_ARG, "lane %d out of range", lane);
  TableLock l;
  int32_t* st = status_of(is_tx);
  if (st[lane] != kBorrowed) return 0;
  st[lane] = kIdle;
  return 1;
}

int fl_monitor_credits(int n_lanes, int own_lane, uint32_t idle_credit, uint32_t* credits_out) {
  if (n_lanes < 1 || n_lanes > kGroups || !credits_out) return fl_set_error(FLH_E_ARG, "bad credit query");
  TableLock l;
  for (int i = 0; i < n_lanes; ++i) credits_out[i] = g_tab->tx_status[i] == kIdle ? idle_credit : 0;
  if (own_lane >= 0 && own_lane < n_lanes && credits_out[own_lane] == 0) credits_out[own_lane] = 1;
  return FLH_OK;
}

// The mask a sender ships with its data (refreshTxUsage, src/fuselink.h:265-267, a placeholder there): bit l set when
// lane l's send side is IDLE in this host's table, the comm's own lane always, and every bit from n_lanes on.
int fl_monitor_tx_mask(int n_lanes, int own_lane, uint32_t* mask_out) {
  if (n_lanes < 1 || n_lanes > kGroups || !mask_out) return fl_set_error(FLH_E_ARG, "bad mask query");
  TableLock l;
  uint32_t mask = ~0u << n_lanes;
  for (int i = 0; i < n_lanes; ++i)
    if (g_tab->tx_status[i] == kIdle || i == own_lane) mask |= 1u << i;
  *mask_out = mask;
  return FLH_OK;
}

// Credits a receiver advertises at a refresh: the query the reference left commented out in refreshRxComm
// (src/fuselink.h:240-243: getIdleNicRx(group, priority, txAvailable), whose mask skips NICs, src/monitor.h:214).
int fl_monitor_rx_credits(int n_lanes, int own_lane, uint32_t idle_credit, uint32_t tx_mask, uint32_t* credits_out) {
  if (n_lanes < 1 || n_lanes > kGroups || !credits_out) return fl_set_error(FLH_E_ARG, "bad credit query");
  TableLock l;
  for (int i = 0; i < n_lanes; ++i) credits_out[i] = g_tab->rx_status[i] == kIdle && ((tx_mask >> i) & 1u) ? idle_credit : 0;
  if (own_lane >= 0 && own_lane < n_lanes && credits_out[own_lane] == 0) credits_out[own_lane] = 1;
  return FLH_OK;
}

}  // extern "C"
