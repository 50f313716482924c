// fl_monitor_main.cc -- the lane-idleness daemon: owns the shared table and ages lanes to IDLE.
//
// Counterpart of the reference's `monitor` binary (FuseLink src/monitor_main.cpp, src/monitor.cpp),
// which as shipped never calls Monitor::initialize() and so dereferences a null table in its loop
// (src/monitor.cpp:30-35, 161).  This one creates the shared memory and the semaphore first, under the
// reference's names, so that the reference's own MonitorClient can attach to it too, then runs the
// reference's loop: every MONITOR_TIMEOUT_US, mark every NIC whose last activity is that old IDLE.
//
//   fuselink-monitor [--seconds S] [--shm NAME] [--sem NAME]      (S <= 0: until SIGTERM / SIGINT)
#include <signal.h>
#include <unistd.h>

#include <chrono>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <thread>

#include "fl_internal.h"
#include "fuselink_net.h"

static char g_err[256];
int fl_set_error(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}
int64_t fl_param(const char*, int64_t dflt) { return dflt; }

extern "C" int fl_monitor_attach_shm(const char* shm_name, const char* sem_name, int create);
extern "C" int fl_monitor_detach(void);

static volatile sig_atomic_t g_stop = 0;
static void on_signal(int) { g_stop = 1; }

int main(int argc, char** argv) {
  double seconds = 10.0;  // the reference's binary runs for 10 s (src/monitor_main.cpp:9)
  const char *shm = nullptr, *sem = nullptr;
  for (int i = 1; i + 1 < argc; i += 2) {
    if (!strcmp(argv[i], "--seconds")) seconds = atof(argv[i + 1]);
    else if (!strcmp(argv[i], "--shm")) shm = argv[i + 1];
    else if (!strcmp(argv[i], "--sem")) sem = argv[i + 1];
  }
  signal(SIGTERM, on_signal);
  signal(SIGINT, on_signal);
  if (fl_monitor_attach_shm(shm, sem, 1) != 0) { fprintf(stderr, "fuselink-monitor: %s\n", g_err); return 1; }
  printf("fuselink-monitor: table up, period %d us\n", FL_NET_MONITOR_TIMEOUT_US);
  fflush(stdout);
  const auto t0 = std::chrono::steady_clock::now();
  while (!g_stop) {
    fl_monitor_tick(fl_monitor_now());
    std::this_thread::sleep_for(std::chrono::microseconds(FL_NET_MONITOR_TIMEOUT_US));  // src/monitor.cpp:190
    if (seconds > 0 && std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count() >= seconds) break;
  }
  fl_monitor_detach();  // clears the running flag, unlinks the shared memory and the semaphore
  return 0;
}
