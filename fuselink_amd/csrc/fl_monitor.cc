// fl_monitor.cc -- lane (virtual NIC) idleness tracking and the credits derived from it.
//
// The reference keeps this state in POSIX shared memory owned by a daemon (FuseLink
// src/monitor.h:47-55, src/monitor.cpp:159-193) and guards every access with a named semaphore.
// Here the table lives in the plugin's process behind a mutex and the clock is an argument, so the
// state machine is deterministic: the transport marks a lane active when it puts traffic on it, a
// tick ages lanes to IDLE after MONITOR_TIMEOUT_US, and the scheduler's credits are read off the
// statuses at each refresh.
#include <chrono>
#include <cstring>
#include <mutex>

#include "fl_internal.h"
#include "fuselink_hip.h"
#include "fuselink_net.h"

namespace {

constexpr int kGroups = FL_NET_MAX_LANES;  // NGROUP with NNIC_PER_GROUP == 1 (src/monitor.h:18-20)
enum : int32_t { kIdle = 0, kBusy = 1, kBorrowed = 2 };  // NicStatus, src/monitor.h:40-44

struct LaneTable {
  int32_t status[2][kGroups];        // [0] rx, [1] tx
  int64_t last_active[2][kGroups];   // microseconds
};

std::mutex g_mu;
LaneTable g_tab = {};
bool g_manual_clock = false;
int64_t g_manual_now = 0;

}  // namespace

extern "C" {

int fl_monitor_set_clock(int manual, int64_t now_us) {
  std::lock_guard<std::mutex> g(g_mu);
  g_manual_clock = manual != 0;
  g_manual_now = now_us;
  return FLH_OK;
}

int64_t fl_monitor_now(void) {
  {
    std::lock_guard<std::mutex> g(g_mu);
    if (g_manual_clock) return g_manual_now;
  }
  return std::chrono::duration_cast<std::chrono::microseconds>(std::chrono::steady_clock::now().time_since_epoch()).count();
}

int fl_monitor_reset(void) {
  std::lock_guard<std::mutex> g(g_mu);
  memset(&g_tab, 0, sizeof(g_tab));
  return FLH_OK;
}

// markNicTxAsActive / markNicRxAsActive (src/monitor.h:236-250)
int fl_monitor_mark_active(int lane, int is_tx, int64_t now_us) {
  if (lane < 0 || lane >= kGroups) return fl_set_error(FLH_E_ARG, "lane %d out of range", lane);
  std::lock_guard<std::mutex> g(g_mu);
  const int d = is_tx ? 1 : 0;
  g_tab.last_active[d][lane] = now_us;
  g_tab.status[d][lane] = kBusy;
  return FLH_OK;
}

int fl_monitor_set_entry(int lane, int is_tx, int32_t status, int64_t last_active_us) {
  if (lane < 0 || lane >= kGroups || status < kIdle || status > kBorrowed) return fl_set_error(FLH_E_ARG, "bad table entry");
  std::lock_guard<std::mutex> g(g_mu);
  g_tab.status[is_tx ? 1 : 0][lane] = status;
  g_tab.last_active[is_tx ? 1 : 0][lane] = last_active_us;
  return FLH_OK;
}

// Monitor::monitorThread body (src/monitor.cpp:164-188): a lane whose last activity is at least the
// timeout old becomes IDLE, whatever it was (BUSY or BORROWED); a younger one keeps its status.
int fl_monitor_tick(int64_t now_us) {
  std::lock_guard<std::mutex> g(g_mu);
  for (int d = 0; d < 2; ++d)
    for (int i = 0; i < kGroups; ++i)
      if (!(g_tab.last_active[d][i] + FL_NET_MONITOR_TIMEOUT_US > now_us)) g_tab.status[d][i] = kIdle;
  return FLH_OK;
}

// getNICStatus (src/monitor.h:226-234), for either direction
int fl_monitor_status(int is_tx, int n_lanes, int32_t* status_out) {
  if (n_lanes < 0 || n_lanes > kGroups || !status_out) return fl_set_error(FLH_E_ARG, "bad status query");
  std::lock_guard<std::mutex> g(g_mu);
  for (int i = 0; i < n_lanes; ++i) status_out[i] = g_tab.status[is_tx ? 1 : 0][i];
  return FLH_OK;
}

// getIdleNicTx / getIdleNicRx (src/monitor.h:191-224).  As written there, the `break` leaves only
// the one-iteration inner loop, so the scan goes on: every idle NIC outside `group` that the mask
// admits is marked BORROWED and the last of them is returned.  exact != 0 stops at the first.
int fl_monitor_idle_pick(int is_tx, int group, int mask, int exact) {
  std::lock_guard<std::mutex> g(g_mu);
  const int d = is_tx ? 1 : 0;
  int found = -1;
  for (int i = 0; i < kGroups; ++i) {
    if (i == group) continue;
    if (!is_tx && (mask & (1 << i)) == 0) continue;  // only the rx query takes a mask (src/monitor.h:214)
    if (g_tab.status[d][i] != kIdle) continue;
    g_tab.status[d][i] = kBorrowed;
    found = i;
    if (exact) break;
  }
  return found;
}

int fl_monitor_credits(int n_lanes, int own_lane, uint32_t idle_credit, uint32_t* credits_out) {
  if (n_lanes < 1 || n_lanes > kGroups || !credits_out) return fl_set_error(FLH_E_ARG, "bad credit query");
  std::lock_guard<std::mutex> g(g_mu);
  for (int l = 0; l < n_lanes; ++l) credits_out[l] = g_tab.status[1][l] == kIdle ? idle_credit : 0;
  if (own_lane >= 0 && own_lane < n_lanes && credits_out[own_lane] == 0) credits_out[own_lane] = 1;
  return FLH_OK;
}

}  // extern "C"
