// plugin_harness.cc -- drives libnccl-net-fuselink.so the way NCCL's proxy threads drive a net plugin:
// dlopen + dlsym of the table, listen / connect / accept, regMr on both sides, then one receiver thread
// posting irecv and polling test and one sender thread issuing isend and polling test, with a bounded
// number of requests in flight.  Verifies the received buffer byte for byte and prints one JSON line.
//
//   plugin_harness <lib.so> [--bytes N] [--request N] [--inflight K] [--iters I] [--host] [--version 6|7|8] [--connections C]
// With --connections C, C connections run concurrently, each with its own pair of proxy threads and buffers.
#include <dlfcn.h>
#include <hip/hip_runtime.h>

#include <atomic>
#include <chrono>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <deque>
#include <string>
#include <thread>
#include <vector>

#include "fuselink_net.h"

static void logger(ncclDebugLogLevel level, unsigned long, const char* file, int line, const char* fmt, ...) {
  if (level != NCCL_LOG_WARN) return;
  va_list ap;
  va_start(ap, fmt);
  fprintf(stderr, "[WARN %s:%d] ", file, line);
  vfprintf(stderr, fmt, ap);
  fprintf(stderr, "\n");
  va_end(ap);
}

#define CHECK(x) do { ncclResult_t r_ = (x); if (r_ != ncclSuccess) { fprintf(stderr, "%s -> ncclResult %d (line %d)\n", #x, (int)r_, __LINE__); exit(2); } } while (0)
#define HIP(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { fprintf(stderr, "%s -> %s\n", #x, hipGetErrorString(e_)); exit(3); } } while (0)

static void run_connection(int ci, ncclNet_v8_t* net8, ncclNet_v7_t* net7, ncclNet_v6_t* net6, size_t bytes, size_t request, int inflight,
                           int iters, int host, int version, double* best_out, double* total_out) {
  if (!host) HIP(hipSetDevice(0));
  const int dev = ci % 2;  // spread the connections over two virtual NICs
  char handle[NCCL_NET_HANDLE_MAXSIZE];
  void *lcomm = nullptr, *scomm = nullptr, *rcomm = nullptr;
  CHECK(net8->listen(dev, handle, &lcomm));
  for (int spin = 0; spin < 1000 && (!scomm || !rcomm); ++spin) {
    if (!scomm) { if (version == 6) CHECK(net6->connect(dev, handle, &scomm)); else CHECK(net8->connect(dev, handle, &scomm, nullptr)); }
    if (!rcomm) { if (version == 6) CHECK(net6->accept(lcomm, &rcomm)); else CHECK(net8->accept(lcomm, &rcomm, nullptr)); }
  }
  if (!scomm || !rcomm) { fprintf(stderr, "connection did not come up\n"); exit(2); }

  std::vector<uint8_t> pattern(bytes);
  uint64_t x = 88172645463325252ull + 7919ull * (uint64_t)ci;
  for (size_t i = 0; i < bytes; ++i) { x ^= x << 13; x ^= x >> 7; x ^= x << 17; pattern[i] = (uint8_t)x; }
  uint8_t *src = nullptr, *dst = nullptr;
  const int type = host ? NCCL_PTR_HOST : NCCL_PTR_CUDA;
  if (host) {
    src = (uint8_t*)malloc(bytes); dst = (uint8_t*)calloc(bytes, 1);
    memcpy(src, pattern.data(), bytes);
  } else {
    HIP(hipSetDevice(0));
    HIP(hipMalloc((void**)&src, bytes)); HIP(hipMalloc((void**)&dst, bytes));
    HIP(hipMemcpy(src, pattern.data(), bytes, hipMemcpyHostToDevice));
    HIP(hipMemset(dst, 0, bytes));
  }
  void *smh = nullptr, *rmh = nullptr;
  if (version == 8) { CHECK(net8->regMr(scomm, src, bytes, type, &smh)); CHECK(net8->regMr(rcomm, dst, bytes, type, &rmh)); }
  else { CHECK(net7->regMr(scomm, src, (int)bytes, type, &smh)); CHECK(net7->regMr(rcomm, dst, (int)bytes, type, &rmh)); }

  const size_t n_req = (bytes + request - 1) / request;
  double best = 1e30, total = 0;
  for (int it = 0; it < iters; ++it) {
    std::atomic<size_t> posted{0};
    auto t0 = std::chrono::steady_clock::now();
    std::thread receiver([&]() {
      if (!host) (void)hipSetDevice(0);
      std::deque<void*> q;
      size_t next = 0, finished = 0;
      while (finished < n_req) {
        if (next < n_req && (int)q.size() < inflight) {
          void* d = dst + next * request;
          int sz = (int)((next + 1) * request <= bytes ? request : bytes - next * request), tag = (int)next;
          void* req = nullptr;
          CHECK(net8->irecv(rcomm, 1, &d, &sz, &tag, &rmh, &req));
          if (req) { q.push_back(req); ++next; posted.store(next, std::memory_order_release); }
        }
        if (!q.empty()) {
          int done = 0, got = -1;
          CHECK(net8->test(q.front(), &done, &got));
          if (done) {
            const size_t k = finished;
            const int want = (int)((k + 1) * request <= bytes ? request : bytes - k * request);
            if (got != want) { fprintf(stderr, "receive %zu reported %d bytes, expected %d\n", k, got, want); exit(4); }
            q.pop_front(); ++finished;
          }
        }
      }
    });
    std::thread sender([&]() {
      if (!host) (void)hipSetDevice(0);
      std::deque<void*> q;
      size_t next = 0, finished = 0;
      while (finished < n_req) {
        if (next < n_req && next < posted.load(std::memory_order_acquire) && (int)q.size() < inflight) {
          int sz = (int)((next + 1) * request <= bytes ? request : bytes - next * request);
          void* req = nullptr;
          CHECK(net8->isend(scomm, src + next * request, sz, (int)next, smh, &req));
          if (req) { q.push_back(req); ++next; }
        }
        if (!q.empty()) {
          int done = 0;
          CHECK(net8->test(q.front(), &done, nullptr));
          if (done) { q.pop_front(); ++finished; }
        }
      }
    });
    sender.join();
    receiver.join();
    double s = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
    total += s;
    if (s < best) best = s;
    std::vector<uint8_t> back(bytes);
    if (host) memcpy(back.data(), dst, bytes); else HIP(hipMemcpy(back.data(), dst, bytes, hipMemcpyDeviceToHost));
    if (memcmp(back.data(), pattern.data(), bytes) != 0) { fprintf(stderr, "connection %d iteration %d: received buffer differs\n", ci, it); exit(5); }
    if (host) memset(dst, 0, bytes); else HIP(hipMemset(dst, 0, bytes));
  }
  CHECK(net8->deregMr(scomm, smh));
  CHECK(net8->deregMr(rcomm, rmh));
  CHECK(net8->closeSend(scomm));
  CHECK(net8->closeRecv(rcomm));
  CHECK(net8->closeListen(lcomm));
  if (host) { free(src); free(dst); } else { HIP(hipFree(src)); HIP(hipFree(dst)); }
  *best_out = best;
  *total_out = total / iters;
}

int main(int argc, char** argv) {
  if (argc < 2) { fprintf(stderr, "usage: %s <libnccl-net-fuselink.so> [options]\n", argv[0]); return 1; }
  size_t bytes = 64u << 20, request = 0;
  int inflight = 4, iters = 5, host = 0, version = 8, connections = 1;
  for (int i = 2; i < argc; ++i) {
    std::string a = argv[i];
    auto val = [&]() { return i + 1 < argc ? strtoull(argv[++i], nullptr, 0) : 0ull; };
    if (a == "--bytes") bytes = val();
    else if (a == "--request") request = val();
    else if (a == "--inflight") inflight = (int)val();
    else if (a == "--iters") iters = (int)val();
    else if (a == "--version") version = (int)val();
    else if (a == "--host") host = 1;
    else if (a == "--connections") connections = (int)val();
  }
  if (!request || request > bytes) request = bytes;
  if (request > 0x7fffffffull) request = 0x40000000ull;  // isend takes an int size (src/extern/nccl_net.h:74)

  void* lib = dlopen(argv[1], RTLD_NOW | RTLD_LOCAL);
  if (!lib) { fprintf(stderr, "dlopen: %s\n", dlerror()); return 1; }
  // the three tables share their leading slots; v8 is used for everything but regMr's size type
  ncclNet_v8_t* net8 = (ncclNet_v8_t*)dlsym(lib, "ncclNetPlugin_v8");
  ncclNet_v7_t* net7 = (ncclNet_v7_t*)dlsym(lib, "ncclNetPlugin_v7");
  ncclNet_v6_t* net6 = (ncclNet_v6_t*)dlsym(lib, "ncclNetPlugin_v6");
  if (!net8 || !net7 || !net6) { fprintf(stderr, "plugin symbols missing\n"); return 1; }
  CHECK(net8->init(logger));
  int ndev = 0;
  CHECK(net8->devices(&ndev));

  std::vector<double> bests(connections, 1e30), totals(connections, 0.0);
  std::vector<std::thread> conns;
  for (int ci = 0; ci < connections; ++ci) conns.emplace_back([&, ci]() { run_connection(ci, net8, net7, net6, bytes, request, inflight, iters, host, version, &bests[ci], &totals[ci]); });
  for (auto& t : conns) t.join();
  double best = 0, total = 0;
  for (int ci = 0; ci < connections; ++ci) { if (bests[ci] > best) best = bests[ci]; total += totals[ci] / connections; }
  const size_t n_req = (bytes + request - 1) / request;
  printf("{\"harness\": \"plugin\", \"name\": \"%s\", \"devices\": %d, \"memory\": \"%s\", \"bytes\": %zu, \"request_bytes\": %zu, \"requests\": %zu, "
         "\"inflight\": %d, \"iters\": %d, \"connections\": %d, \"best_s\": %.9f, \"mean_s\": %.9f, \"GBps_4N_best\": %.1f, \"bit_exact\": true}\n",
         net8->name, ndev, host ? "host" : "device", bytes, request, n_req, inflight, iters, connections, best, total, 4.0 * bytes * connections / best / 1e9);
  return 0;
}
