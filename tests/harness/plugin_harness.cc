// plugin_harness.cc -- drives libnccl-net-fuselink.so the way NCCL's proxy threads drive a net plugin:
// dlopen + dlsym of the table, listen / connect / accept, regMr on both sides, then one receiver thread
// posting irecv and polling test and one sender thread issuing isend and polling test, with a bounded
// number of requests in flight.  Verifies the received buffer byte for byte and prints one JSON line.
//
//   plugin_harness <lib.so> [--bytes N] [--request N] [--inflight K] [--iters I] [--host] [--version 6|7|8] [--connections C]
//                  [--handoff batch,blocks_per_req,layers,kv_heads,block_size,head_dim] [--two-process] [--side-streams S]
// With --side-streams S, a thread of the harness keeps S more HIP streams of the process busy with small fills while the
// connections run -- the application's own compute streams beside the plugin's -- and reports how long a fill took from
// its launch to its completion (mean and worst).  A process has fewer hardware queues than that many streams, so some of
// them share a queue with the plugin's streams: what they wait for is how long the plugin's kernels hold a queue.
// With --two-process the receiver is a child process forked before either side has touched the GPU or loaded the plugin:
// the child listens and sends the 128-byte handle to the parent over a socket pair (NCCL's bootstrap does that between
// ranks), the parent connects with it, and from then on the two processes share nothing but what the plugin itself set up
// behind the handle (NCCL_FUSELINK_WIRE=shm is set for both).  The child checks what it received and reports through its
// exit status.  With --handoff as well, the five messages of the hand-off group cross the process boundary, each a
// buffer and a registration of its own on either side.
// With --connections C, C connections run concurrently, each with its own pair of proxy threads and buffers; every
// iteration starts on all of them together and is timed from the first start to the last finish, and the received
// buffers are compared only once all connections have finished it.
// With --handoff the message is the prefill -> decode hand-off of the reference's serving experiment
// (FuseLink experiments/serving/model.hh:280-309): one group of five sends on one connection -- the context output
// (int64 per request), the K cache, the V cache, the block table (int64 per request and block) and the allocated-block
// counts (int64 per request) -- each cut into --request sized pieces as NCCL's proxy would.
#include <dlfcn.h>
#include <hip/hip_runtime.h>
#include <signal.h>
#include <sys/socket.h>
#include <sys/wait.h>
#include <unistd.h>

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

// all connections meet here before and after the transfers of an iteration
struct Barrier {
  std::atomic<int> arrived{0}, generation{0};
  int parties = 1;
  void wait() {
    const int gen = generation.load(std::memory_order_acquire);
    if (arrived.fetch_add(1, std::memory_order_acq_rel) + 1 == parties) {
      arrived.store(0, std::memory_order_relaxed);
      generation.store(gen + 1, std::memory_order_release);
    } else {
      while (generation.load(std::memory_order_acquire) == gen) std::this_thread::yield();
    }
  }
};
typedef std::chrono::steady_clock::time_point TimePoint;

static void run_connection(int ci, ncclNet_v8_t* net8, ncclNet_v7_t* net7, ncclNet_v6_t* net6, const std::vector<size_t>& sizes, size_t request, int inflight,
                           int iters, int host, int version, Barrier* barrier, TimePoint* starts, TimePoint* ends) {
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

  // the messages of one group, sent in order over this connection
  struct Msg { size_t bytes; uint8_t *src, *dst; void *smh, *rmh; std::vector<uint8_t> pattern; };
  std::vector<Msg> msgs(sizes.size());
  const int type = host ? NCCL_PTR_HOST : NCCL_PTR_CUDA;
  uint64_t x = 88172645463325252ull + 7919ull * (uint64_t)ci;
  size_t bytes = 0;
  for (size_t m = 0; m < sizes.size(); ++m) {
    Msg& g = msgs[m];
    g.bytes = sizes[m];
    bytes += g.bytes;
    g.pattern.resize(g.bytes);
    for (size_t i = 0; i < g.bytes; ++i) { x ^= x << 13; x ^= x >> 7; x ^= x << 17; g.pattern[i] = (uint8_t)x; }
    if (host) {
      g.src = (uint8_t*)malloc(g.bytes); g.dst = (uint8_t*)calloc(g.bytes, 1);
      memcpy(g.src, g.pattern.data(), g.bytes);
    } else {
      HIP(hipSetDevice(0));
      HIP(hipMalloc((void**)&g.src, g.bytes)); HIP(hipMalloc((void**)&g.dst, g.bytes));
      HIP(hipMemcpy(g.src, g.pattern.data(), g.bytes, hipMemcpyHostToDevice));
      HIP(hipMemset(g.dst, 0, g.bytes));
    }
    if (version == 8) { CHECK(net8->regMr(scomm, g.src, g.bytes, type, &g.smh)); CHECK(net8->regMr(rcomm, g.dst, g.bytes, type, &g.rmh)); }
    else { CHECK(net7->regMr(scomm, g.src, (int)g.bytes, type, &g.smh)); CHECK(net7->regMr(rcomm, g.dst, (int)g.bytes, type, &g.rmh)); }
  }
  // request k of the group: which message, where in it, how long
  struct Piece { int msg; size_t off; int len; };
  std::vector<Piece> pieces;
  for (size_t m = 0; m < msgs.size(); ++m)
    for (size_t off = 0; off < msgs[m].bytes; off += request)
      pieces.push_back({(int)m, off, (int)(msgs[m].bytes - off < request ? msgs[m].bytes - off : request)});
  const size_t n_req = pieces.size();
  for (int it = 0; it < iters; ++it) {
    std::atomic<size_t> posted{0};
    barrier->wait();
    starts[it] = std::chrono::steady_clock::now();
    std::thread receiver([&]() {
      if (!host) (void)hipSetDevice(0);
      std::deque<void*> q;
      size_t next = 0, finished = 0;
      while (finished < n_req) {
        if (next < n_req && (int)q.size() < inflight) {
          const Piece& pc = pieces[next];
          void* d = msgs[pc.msg].dst + pc.off;
          int sz = pc.len, tag = (int)next;
          void* req = nullptr;
          CHECK(net8->irecv(rcomm, 1, &d, &sz, &tag, &msgs[pc.msg].rmh, &req));
          if (req) { q.push_back(req); ++next; posted.store(next, std::memory_order_release); }
        }
        if (!q.empty()) {
          int done = 0, got = -1;
          CHECK(net8->test(q.front(), &done, &got));
          if (done) {
            const int want = pieces[finished].len;
            if (got != want) { fprintf(stderr, "receive %zu reported %d bytes, expected %d\n", finished, got, want); exit(4); }
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
          const Piece& pc = pieces[next];
          void* req = nullptr;
          CHECK(net8->isend(scomm, msgs[pc.msg].src + pc.off, pc.len, (int)next, msgs[pc.msg].smh, &req));
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
    ends[it] = std::chrono::steady_clock::now();
    barrier->wait();
    for (size_t m = 0; m < msgs.size(); ++m) {
      Msg& g = msgs[m];
      std::vector<uint8_t> back(g.bytes);
      if (host) memcpy(back.data(), g.dst, g.bytes); else HIP(hipMemcpy(back.data(), g.dst, g.bytes, hipMemcpyDeviceToHost));
      if (memcmp(back.data(), g.pattern.data(), g.bytes) != 0) { fprintf(stderr, "connection %d iteration %d message %zu: received buffer differs\n", ci, it, m); exit(5); }
      if (host) memset(g.dst, 0, g.bytes); else HIP(hipMemset(g.dst, 0, g.bytes));
    }
  }
  for (Msg& g : msgs) {
    CHECK(net8->deregMr(scomm, g.smh));
    CHECK(net8->deregMr(rcomm, g.rmh));
  }
  CHECK(net8->closeSend(scomm));
  CHECK(net8->closeRecv(rcomm));
  CHECK(net8->closeListen(lcomm));
  for (Msg& g : msgs) { if (host) { free(g.src); free(g.dst); } else { HIP(hipFree(g.src)); HIP(hipFree(g.dst)); } }
  (void)bytes;
}

// ---- the application's own streams beside the plugin's ----------------------------------------------------------------
struct SideStreams {
  int n = 0;
  std::atomic<bool> stop{false};
  std::thread th;
  double mean_us = 0, max_us = 0;
  long ops = 0;
  void start(int streams) {
    n = streams;
    th = std::thread([this]() {
      HIP(hipSetDevice(0));
      std::vector<hipStream_t> st(n);
      std::vector<void*> buf(n);
      for (int i = 0; i < n; ++i) { HIP(hipStreamCreateWithFlags(&st[i], hipStreamNonBlocking)); HIP(hipMalloc(&buf[i], 4096)); }
      double sum = 0;
      while (!stop.load(std::memory_order_acquire)) {
        for (int i = 0; i < n; ++i) {
          const auto t0 = std::chrono::steady_clock::now();
          HIP(hipMemsetAsync(buf[i], i, 4096, st[i]));
          HIP(hipStreamSynchronize(st[i]));
          const double us = std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count();
          sum += us;
          if (us > max_us) max_us = us;
          ++ops;
        }
        std::this_thread::sleep_for(std::chrono::microseconds(50));
      }
      mean_us = ops ? sum / ops : 0;
      for (int i = 0; i < n; ++i) { HIP(hipStreamDestroy(st[i])); HIP(hipFree(buf[i])); }
    });
  }
  void finish() {
    if (!n) return;
    stop.store(true, std::memory_order_release);
    th.join();
  }
};

// ---- two processes ------------------------------------------------------------------------------------------------
static void fill_pattern(std::vector<uint8_t>& p, int iteration) {
  uint64_t x = 88172645463325252ull + 104729ull * (uint64_t)iteration;
  for (size_t i = 0; i < p.size(); ++i) { x ^= x << 13; x ^= x >> 7; x ^= x << 17; p[i] = (uint8_t)x; }
}
static void sock_write(int fd, const void* p, size_t n) {
  if (write(fd, p, n) != (ssize_t)n) { fprintf(stderr, "socket write failed\n"); exit(6); }
}
// blocking read with a deadline, so that neither process outlives the other by more than that
static void sock_read(int fd, void* p, size_t n, double seconds) {
  const auto t0 = std::chrono::steady_clock::now();
  size_t got = 0;
  while (got < n) {
    ssize_t k = recv(fd, (char*)p + got, n - got, MSG_DONTWAIT);
    if (k > 0) { got += (size_t)k; continue; }
    if (k == 0) { fprintf(stderr, "the other process closed its end\n"); exit(6); }
    if (std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count() > seconds) { fprintf(stderr, "timed out waiting for the other process\n"); exit(6); }
    usleep(200);
  }
}
static ncclNet_v8_t* open_plugin(const char* path) {
  void* lib = dlopen(path, RTLD_NOW | RTLD_LOCAL);
  if (!lib) { fprintf(stderr, "dlopen: %s\n", dlerror()); exit(1); }
  ncclNet_v8_t* net8 = (ncclNet_v8_t*)dlsym(lib, "ncclNetPlugin_v8");
  if (!net8) { fprintf(stderr, "plugin symbols missing\n"); exit(1); }
  CHECK(net8->init(logger));
  int ndev = 0;
  CHECK(net8->devices(&ndev));
  return net8;
}
// NCCL_FUSELINK_TRACE=2 and FL_TIMELINE_OUT=<file>: the entry-point timeline of this process, one event per line
// (nanoseconds of the machine's monotonic clock, thread, event, value), into <file><suffix>
static void dump_timeline(const char* lib_path, const char* suffix) {
  const char* tr = getenv("NCCL_FUSELINK_TRACE");
  const char* tl_out = getenv("FL_TIMELINE_OUT");
  if (!tr || atoi(tr) < 2 || !tl_out) return;
  void* lib = dlopen(lib_path, RTLD_NOW | RTLD_LOCAL);
  typedef int (*timeline_fn)(void*, int);
  timeline_fn timeline = lib ? (timeline_fn)dlsym(lib, "fl_net_timeline") : nullptr;
  if (!timeline) return;
  struct Ev { int64_t ns; uint32_t thread, event; uint64_t value; };
  std::vector<Ev> ev(65536);
  const int n = timeline(ev.data(), (int)ev.size());
  FILE* f = fopen((std::string(tl_out) + suffix).c_str(), "w");
  if (!f) return;
  for (int i = 0; i < n && i < (int)ev.size(); ++i) fprintf(f, "%lld %u %u %llu\n", (long long)ev[i].ns, ev[i].thread, ev[i].event, (unsigned long long)ev[i].value);
  fclose(f);
}

static const double kDeadline = 90.0;   // seconds any one wait may last
struct Deadline {
  std::chrono::steady_clock::time_point t0 = std::chrono::steady_clock::now();
  void check(const char* what) const {
    if (std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count() > kDeadline) { fprintf(stderr, "timed out: %s\n", what); exit(6); }
  }
};

// the requests of a group of messages, in order: message, offset in it, length
struct WirePiece { int msg; size_t off; int len; };
static std::vector<WirePiece> wire_pieces(const std::vector<size_t>& sizes, size_t request) {
  std::vector<WirePiece> pieces;
  for (size_t m = 0; m < sizes.size(); ++m)
    for (size_t off = 0; off < sizes[m]; off += request)
      pieces.push_back({(int)m, off, (int)(sizes[m] - off < request ? sizes[m] - off : request)});
  return pieces;
}

static int receiver_process(const char* path, int sock, const std::vector<size_t>& sizes, size_t request, int inflight, int iters) {
  ncclNet_v8_t* net = open_plugin(path);
  char handle[NCCL_NET_HANDLE_MAXSIZE];
  void *lcomm = nullptr, *rcomm = nullptr;
  CHECK(net->listen(0, handle, &lcomm));
  sock_write(sock, handle, sizeof(handle));
  for (Deadline d; !rcomm; d.check("accept")) { CHECK(net->accept(lcomm, &rcomm, nullptr)); if (!rcomm) usleep(100); }
  HIP(hipSetDevice(0));
  size_t bytes = 0;
  std::vector<uint8_t*> dst(sizes.size(), nullptr);
  std::vector<void*> mh(sizes.size(), nullptr);
  std::vector<size_t> base(sizes.size(), 0);
  for (size_t m = 0; m < sizes.size(); ++m) {   // every message is a buffer and a registration of its own
    base[m] = bytes;
    bytes += sizes[m];
    HIP(hipMalloc((void**)&dst[m], sizes[m]));
    HIP(hipMemset(dst[m], 0, sizes[m]));
    CHECK(net->regMr(rcomm, dst[m], sizes[m], NCCL_PTR_CUDA, &mh[m]));
  }
  const std::vector<WirePiece> pieces = wire_pieces(sizes, request);
  const size_t n_req = pieces.size();
  std::vector<uint8_t> pattern(bytes), back(bytes);
  for (int it = 0; it < iters; ++it) {
    char go = 0;
    sock_read(sock, &go, 1, kDeadline);
    std::deque<void*> q;
    size_t next = 0, finished = 0;
    Deadline d;
    while (finished < n_req) {
      if (next < n_req && (int)q.size() < inflight) {
        const WirePiece& pc = pieces[next];
        void* p = dst[pc.msg] + pc.off;
        int sz = pc.len, tag = (int)next;
        void* req = nullptr;
        CHECK(net->irecv(rcomm, 1, &p, &sz, &tag, &mh[pc.msg], &req));
        if (req) { q.push_back(req); ++next; }
      }
      if (!q.empty()) {
        int done = 0, got = -1;
        CHECK(net->test(q.front(), &done, &got));
        if (done) {
          if (got != pieces[finished].len) { fprintf(stderr, "receive %zu reported %d bytes, expected %d\n", finished, got, pieces[finished].len); return 4; }
          q.pop_front(); ++finished;
        }
      }
      d.check("receives");
    }
    fill_pattern(pattern, it);
    for (size_t m = 0; m < sizes.size(); ++m) {
      HIP(hipMemcpy(back.data() + base[m], dst[m], sizes[m], hipMemcpyDeviceToHost));
      if (memcmp(back.data() + base[m], pattern.data() + base[m], sizes[m]) != 0) {
        size_t at = 0;
        while (at < sizes[m] && back[base[m] + at] == pattern[base[m] + at]) ++at;
        fprintf(stderr, "iteration %d, message %zu: the received buffer differs from what was sent, first at byte %zu\n", it, m, at);
        return 5;
      }
      HIP(hipMemset(dst[m], 0, sizes[m]));
    }
    char ok = 1;
    sock_write(sock, &ok, 1);
  }
  char bye = 0;
  sock_read(sock, &bye, 1, kDeadline);   // the sender has closed its comm: the landing windows may go
  for (size_t m = 0; m < sizes.size(); ++m) CHECK(net->deregMr(rcomm, mh[m]));
  CHECK(net->closeRecv(rcomm));
  CHECK(net->closeListen(lcomm));
  for (uint8_t* p : dst) HIP(hipFree(p));
  dump_timeline(path, ".receiver");
  return 0;
}

static int sender_process(const char* path, int sock, pid_t child, const std::vector<size_t>& sizes, size_t request, int inflight, int iters, int handoff) {
  ncclNet_v8_t* net = open_plugin(path);
  char handle[NCCL_NET_HANDLE_MAXSIZE];
  sock_read(sock, handle, sizeof(handle), kDeadline);
  void* scomm = nullptr;
  for (Deadline d; !scomm; d.check("connect")) { CHECK(net->connect(1, handle, &scomm, nullptr)); if (!scomm) usleep(100); }
  HIP(hipSetDevice(0));
  size_t bytes = 0;
  std::vector<uint8_t*> src(sizes.size(), nullptr);
  std::vector<void*> mh(sizes.size(), nullptr);
  std::vector<size_t> base(sizes.size(), 0);
  for (size_t m = 0; m < sizes.size(); ++m) {
    base[m] = bytes;
    bytes += sizes[m];
    HIP(hipMalloc((void**)&src[m], sizes[m]));
    CHECK(net->regMr(scomm, src[m], sizes[m], NCCL_PTR_CUDA, &mh[m]));
  }
  const std::vector<WirePiece> pieces = wire_pieces(sizes, request);
  const size_t n_req = pieces.size();
  std::vector<uint8_t> pattern(bytes);
  double best = 1e30, total = 0;
  for (int it = 0; it < iters; ++it) {
    fill_pattern(pattern, it);
    for (size_t m = 0; m < sizes.size(); ++m) HIP(hipMemcpy(src[m], pattern.data() + base[m], sizes[m], hipMemcpyHostToDevice));
    char go = 1;
    const auto t0 = std::chrono::steady_clock::now();
    sock_write(sock, &go, 1);
    std::deque<void*> q;
    size_t next = 0, finished = 0;
    Deadline d;
    while (finished < n_req) {
      if (next < n_req && (int)q.size() < inflight) {
        const WirePiece& pc = pieces[next];
        void* req = nullptr;
        CHECK(net->isend(scomm, src[pc.msg] + pc.off, pc.len, (int)next, mh[pc.msg], &req));   // no request: the receive is not posted yet
        if (req) { q.push_back(req); ++next; }
      }
      if (!q.empty()) {
        int done = 0;
        CHECK(net->test(q.front(), &done, nullptr));
        if (done) { q.pop_front(); ++finished; }
      }
      d.check("sends");
    }
    const double sec = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
    if (sec < best) best = sec;
    total += sec / iters;
    char ok = 0;
    sock_read(sock, &ok, 1, kDeadline);   // the receiver has compared the buffers
  }
  for (size_t m = 0; m < sizes.size(); ++m) CHECK(net->deregMr(scomm, mh[m]));
  CHECK(net->closeSend(scomm));
  for (uint8_t* p : src) HIP(hipFree(p));
  dump_timeline(path, ".sender");
  char bye = 1;
  sock_write(sock, &bye, 1);
  int status = 0;
  Deadline d;
  while (waitpid(child, &status, WNOHANG) == 0) { usleep(1000); d.check("the receiver's exit"); }
  if (!WIFEXITED(status) || WEXITSTATUS(status) != 0) { fprintf(stderr, "the receiver process failed (status 0x%x)\n", status); return 5; }
  printf("{\"harness\": \"plugin_two_process\", \"name\": \"%s\", \"memory\": \"device\", \"group\": \"%s\", \"messages\": %zu, \"bytes\": %zu, \"request_bytes\": %zu, \"requests\": %zu, "
         "\"inflight\": %d, \"iters\": %d, \"best_s\": %.9f, \"mean_s\": %.9f, \"GBps_payload_best\": %.1f, \"bit_exact\": true}\n",
         net->name, handoff ? "kv_handoff" : "one message", sizes.size(), bytes, request, n_req, inflight, iters, best, total, (double)bytes / best / 1e9);
  return 0;
}

static int run_two_processes(const char* path, const std::vector<size_t>& sizes, size_t request, int inflight, int iters, int handoff) {
  setenv("NCCL_FUSELINK_WIRE", "shm", 1);
  int sv[2];
  if (socketpair(AF_UNIX, SOCK_STREAM, 0, sv) != 0) { perror("socketpair"); return 1; }
  fflush(stdout);
  fflush(stderr);
  const pid_t child = fork();   // before anything here has loaded the plugin or called HIP
  if (child < 0) { perror("fork"); return 1; }
  if (child == 0) {
    close(sv[0]);
    const int rc = receiver_process(path, sv[1], sizes, request, inflight, iters);
    fflush(stderr);
    _exit(rc);
  }
  close(sv[1]);
  signal(SIGPIPE, SIG_IGN);
  return sender_process(path, sv[0], child, sizes, request, inflight, iters, handoff);
}

int main(int argc, char** argv) {
  if (argc < 2) { fprintf(stderr, "usage: %s <libnccl-net-fuselink.so> [options]\n", argv[0]); return 1; }
  size_t bytes = 64u << 20, request = 0;
  int inflight = 4, iters = 5, host = 0, version = 8, connections = 1, handoff = 0, two_process = 0, side_streams = 0;
  long long ho[6] = {0, 0, 0, 0, 0, 0};
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
    else if (a == "--two-process") two_process = 1;
    else if (a == "--side-streams") side_streams = (int)val();
    else if (a == "--handoff" && i + 1 < argc) {
      if (sscanf(argv[++i], "%lld,%lld,%lld,%lld,%lld,%lld", &ho[0], &ho[1], &ho[2], &ho[3], &ho[4], &ho[5]) != 6) { fprintf(stderr, "--handoff takes six numbers\n"); return 1; }
      handoff = 1;
    }
  }
  std::vector<size_t> sizes{bytes};
  if (handoff) {
    // experiments/serving/model.hh:198-201, 283: cache bytes = sizeof(half) * blocks * layers * kv_heads * block_size * head_dim
    const size_t batch = (size_t)ho[0], blocks = (size_t)(ho[0] * ho[1]);
    const size_t cache = 2ull * blocks * (size_t)ho[2] * (size_t)ho[3] * (size_t)ho[4] * (size_t)ho[5];
    sizes = {8 * batch, cache, cache, 8 * blocks, 8 * batch};   // the five sends of model.hh:286-309, in order
    bytes = 0;
    for (size_t b : sizes) bytes += b;
  }
  if (!request || request > bytes) request = bytes;
  if (request > 0x7fffffffull) request = 0x40000000ull;  // isend takes an int size (src/extern/nccl_net.h:74)

  if (two_process) {
    if (host || connections != 1) { fprintf(stderr, "--two-process runs one connection with device memory\n"); return 1; }
    return run_two_processes(argv[1], sizes, request, inflight, iters, handoff);
  }

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

  Barrier barrier;
  barrier.parties = connections;
  std::vector<std::vector<TimePoint>> starts(connections, std::vector<TimePoint>(iters)), ends(connections, std::vector<TimePoint>(iters));
  SideStreams side;
  if (side_streams > 0 && !host) side.start(side_streams);
  std::vector<std::thread> conns;
  for (int ci = 0; ci < connections; ++ci)
    conns.emplace_back([&, ci]() { run_connection(ci, net8, net7, net6, sizes, request, inflight, iters, host, version, &barrier, starts[ci].data(), ends[ci].data()); });
  for (auto& t : conns) t.join();
  side.finish();
  // an iteration lasts from the first connection's start to the last connection's finish
  double best = 1e30, total = 0;
  for (int it = 0; it < iters; ++it) {
    TimePoint first = starts[0][it], last = ends[0][it];
    for (int ci = 1; ci < connections; ++ci) { if (starts[ci][it] < first) first = starts[ci][it]; if (ends[ci][it] > last) last = ends[ci][it]; }
    const double sec = std::chrono::duration<double>(last - first).count();
    if (sec < best) best = sec;
    total += sec / iters;
  }
  size_t n_req = 0;
  for (size_t b : sizes) n_req += (b + request - 1) / request;
  if (handoff)
    printf("{\"harness\": \"kv_handoff\", \"batch\": %lld, \"blocks\": %lld, \"layers\": %lld, \"kv_heads\": %lld, \"block_size\": %lld, \"head_dim\": %lld, "
           "\"cache_bytes_each\": %zu, \"comm_volume_bytes\": %zu, \"best_s\": %.9f, \"GBps_volume_over_time\": %.1f}\n",
           ho[0], ho[0] * ho[1], ho[2], ho[3], ho[4], ho[5], sizes[1], bytes, best, (double)bytes * connections / best / 1e9);
  printf("{\"harness\": \"plugin\", \"name\": \"%s\", \"devices\": %d, \"memory\": \"%s\", \"bytes\": %zu, \"request_bytes\": %zu, \"requests\": %zu, "
         "\"inflight\": %d, \"iters\": %d, \"connections\": %d, \"best_s\": %.9f, \"mean_s\": %.9f, \"GBps_4N_best\": %.1f, \"bit_exact\": true}\n",
         net8->name, ndev, host ? "host" : "device", bytes, request, n_req, inflight, iters, connections, best, total, 4.0 * bytes * connections / best / 1e9);
  if (side.n)
    printf("{\"harness\": \"side_streams\", \"streams\": %d, \"fills\": %ld, \"fill_us_mean\": %.1f, \"fill_us_max\": %.1f}\n", side.n, side.ops, side.mean_us, side.max_us);
  // NCCL_FUSELINK_TRACE=1: where the host's time went, summed over all proxy threads
  typedef int (*host_stats_fn)(int64_t*, int64_t*, int);
  host_stats_fn host_stats = (host_stats_fn)dlsym(lib, "fl_net_host_stats");
  const char* tr = getenv("NCCL_FUSELINK_TRACE");
  if (host_stats && tr && atoi(tr) > 0) {
    int64_t calls[16] = {0}, ns[16] = {0};
    host_stats(calls, ns, 16);
    const double reqs = (double)n_req * connections * iters;
    printf("{\"harness\": \"host_trace\", \"requests\": %.0f, \"isend_calls\": %lld, \"isend_us\": %.1f, \"irecv_calls\": %lld, \"irecv_us\": %.1f, "
           "\"test_calls\": %lld, \"test_us\": %.1f, \"tests_done\": %lld, \"flush_passes\": %lld, \"flush_us\": %.1f, \"launch_pairs\": %lld, \"launch_us\": %.1f, "
           "\"requests_per_launch\": %.2f, \"launch_us_per_pair\": %.2f, \"engine_submits\": %lld, \"engine_submit_us\": %.1f, \"engine_starts\": %lld, \"engine_start_us\": %.1f}\n",
           reqs, (long long)calls[0], ns[0] / 1e3, (long long)calls[1], ns[1] / 1e3, (long long)calls[2], ns[2] / 1e3, (long long)calls[3],
           (long long)calls[4], ns[4] / 1e3, (long long)calls[5], ns[5] / 1e3, calls[5] ? (double)calls[6] / calls[5] : 0.0, calls[5] ? ns[5] / 1e3 / calls[5] : 0.0,
           (long long)calls[7], ns[7] / 1e3, (long long)calls[8], ns[8] / 1e3);
  }
  // NCCL_FUSELINK_TRACE=2: the timeline of the entry-point events, one line per event, into the file named by FL_TIMELINE_OUT
  typedef int (*timeline_fn)(void*, int);
  timeline_fn timeline = (timeline_fn)dlsym(lib, "fl_net_timeline");
  const char* tl_out = getenv("FL_TIMELINE_OUT");
  if (timeline && tr && atoi(tr) > 1 && tl_out) {
    struct Ev { int64_t ns; uint32_t thread, event; uint64_t value; };
    std::vector<Ev> ev(65536);
    const int n = timeline(ev.data(), (int)ev.size());
    FILE* f = fopen(tl_out, "w");
    if (f) {
      for (int i = 0; i < n && i < (int)ev.size(); ++i)
        fprintf(f, "%lld %u %u %llu\n", (long long)(ev[i].ns - ev[0].ns), ev[i].thread, ev[i].event, (unsigned long long)ev[i].value);
      fclose(f);
    }
  }
  return 0;
}
