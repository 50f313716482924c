// ref_monitor_shim.cc -- thin C entry points over the REFERENCE's own MonitorClient, compiled from
// src/monitor.h where it lies in the FuseLink tree (never copied).  TEST INFRASTRUCTURE ONLY: it
// exists so that the restated monitor state machine in fl_oracle.c can be checked against the real
// code.  The shim plays the daemon's part of creating the POSIX shared memory and the named
// semaphore (Monitor::setupSharedMemory lives in monitor.cpp, which needs libibverbs headers that
// this image lacks), then drives the unmodified client class.
#include <monitor.h>

#include <cstddef>
#include <cstring>

namespace {
MonitorClient* g_client = nullptr;
SharedMemory* g_shm = nullptr;
int g_fd = -1;
sem_t* g_sem = SEM_FAILED;
}  // namespace

extern "C" {

int ref_mon_open() {
  if (g_client) return 0;
  shm_unlink(SHM_NAME);
  sem_unlink(SEM_NAME);
  g_fd = shm_open(SHM_NAME, O_CREAT | O_RDWR, 0666);
  if (g_fd < 0) return -1;
  if (ftruncate(g_fd, sizeof(SharedMemory)) != 0) return -2;
  g_shm = static_cast<SharedMemory*>(mmap(nullptr, sizeof(SharedMemory), PROT_READ | PROT_WRITE, MAP_SHARED, g_fd, 0));
  if (g_shm == MAP_FAILED) return -3;
  std::memset(static_cast<void*>(g_shm), 0, sizeof(SharedMemory));
  g_sem = sem_open(SEM_NAME, O_CREAT, 0666, 1);
  if (g_sem == SEM_FAILED) return -4;
  try {
    g_client = new MonitorClient();
  } catch (...) {
    return -5;
  }
  return 0;
}

// attach the reference's client to shared memory that somebody else (a daemon) created
int ref_mon_attach() {
  if (g_client) return 0;
  try {
    g_client = new MonitorClient();
  } catch (...) {
    return -5;
  }
  return 0;
}

void ref_mon_detach() {
  delete g_client;
  g_client = nullptr;
}

void ref_mon_close() {
  delete g_client;
  g_client = nullptr;
  if (g_shm && g_shm != MAP_FAILED) munmap(g_shm, sizeof(SharedMemory));
  g_shm = nullptr;
  if (g_fd >= 0) close(g_fd);
  g_fd = -1;
  if (g_sem != SEM_FAILED) sem_close(g_sem);
  g_sem = SEM_FAILED;
  shm_unlink(SHM_NAME);
  sem_unlink(SEM_NAME);
}

// raw access to the shared state, so a test can set up a pattern and read the side effects back
void ref_mon_set(int tx, int group, int nic, int status, long long ts) {
  if (tx) { g_shm->nic_tx_statuses[group][nic] = static_cast<NicStatus>(status); g_shm->nic_tx_last_active_ts[group][nic] = ts; }
  else    { g_shm->nic_rx_statuses[group][nic] = static_cast<NicStatus>(status); g_shm->nic_rx_last_active_ts[group][nic] = ts; }
}
int ref_mon_get_status(int tx, int group, int nic) {
  return tx ? g_shm->nic_tx_statuses[group][nic] : g_shm->nic_rx_statuses[group][nic];
}
long long ref_mon_get_ts(int tx, int group, int nic) {
  return tx ? g_shm->nic_tx_last_active_ts[group][nic] : g_shm->nic_rx_last_active_ts[group][nic];
}

int ref_mon_idle_pick_tx(int group, int primary) { return g_client->getIdleNicTx(group, primary); }
int ref_mon_idle_pick_rx(int group, int primary, int mask) { return g_client->getIdleNicRx(group, primary, mask); }
void ref_mon_mark_tx(int group, int nic) { g_client->markNicTxAsActive(group, nic); }
void ref_mon_mark_rx(int group, int nic) { g_client->markNicRxAsActive(group, nic); }
void ref_mon_status(int n, int* out) {
  NicStatus st[MAX_NIC_NUM];
  g_client->getNICStatus(n, st);
  for (int i = 0; i < n; ++i) out[i] = st[i];
}
long long ref_mon_now() { return get_timestamp(); }

// constants and layout of the reference header
int ref_mon_const(int which) {
  switch (which) {
    case 0: return MAX_NIC_NUM;
    case 1: return NNIC_PER_GROUP;
    case 2: return NGROUP;
    case 3: return NCHANNELS_PER_NIC;
    case 4: return MONITOR_TIMEOUT_US;
    case 5: return NIC_STATUS_IDLE;
    case 6: return NIC_STATUS_BUSY;
    case 7: return NIC_STATUS_BORROWED;
    case 8: return static_cast<int>(sizeof(SharedMemory));
    case 9: return static_cast<int>(offsetof(SharedMemory, nic_tx_statuses));
    case 10: return static_cast<int>(offsetof(SharedMemory, nic_rx_statuses));
    case 11: return static_cast<int>(offsetof(SharedMemory, nic_tx_last_active_ts));
    case 12: return static_cast<int>(offsetof(SharedMemory, nic_rx_last_active_ts));
    case 13: return static_cast<int>(offsetof(SharedMemory, running));
  }
  return -1;
}

}  // extern "C"
