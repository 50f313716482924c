// fl_plugin.cc -- the ncclNet plugin tables (v8, v7, v6) over an in-process loopback wire.
//
// What a request does here, next to what the reference does (FuseLink src/plugin.cc):
//   irecv  posts a descriptor into the sender's FIFO: address, size, tag, the slot index handshake
//          idx = tail+1, the lane decision `fuselink_offset`, and -- in the padding the reference
//          leaves unused -- the receiver's credit row (plugin.cc:1616-1677, 1679-1766).  The lane
//          decision is refreshed every N_FINISHED_BATCH completions and only when nothing posted is
//          outstanding (plugin.cc:1700-1716).
//   isend  matches the FIFO head (plugin.cc:1510-1517), checks sizes (1555-1570), splits the request
//          over QPs in 128-byte-aligned pieces (1467-1495) and then, instead of posting RDMA writes
//          out of a remapped buffer, queues on the connection's HIP stream, per wave of chunks:
//          striping kernel (chunk -> lane scheduling folded in; user buffer -> lane staging windows)
//          -> reassembly kernel (windows -> the posted receive buffer).  The reassembly launch plays the part of the
//          RDMA write landing at the receiver; its completion event is the receive completion.
//          The launches are not made inside isend: matched sends of ALL connections that stage on one GPU wait
//          in one queue (as the reference's channels share one set of per-NIC lane comms, fuselink.h:271-272,
//          plugin.cc:727-753) until a test finds the GPU's queue short of work (or until NCCL_FUSELINK_BATCH of
//          them wait), and go out together: up to 32 requests in one launch pair, the requests of a connection
//          between two refreshes as one message under that connection's credit row, which is what keeps the
//          cost of a launch from bounding the request rate at NCCL's 512 KiB steps.
//   test   launches what waits, reads the completion word that the reassembly kernel's last workgroup stores
//          (the completion queue of plugin.cc:1801-1955) and, unlike the reference, reports the byte count of a receive.
// Staging windows are HIP-VMM mappings from the unit pool, one per lane per GPU, shared by every connection
// that stages there, bound when device memory is first registered on a send side and reused launch after launch.
#include <fcntl.h>
#include <hip/hip_runtime.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <ctime>
#include <deque>
#include <map>
#include <mutex>
#include <new>
#include <thread>
#include <vector>

#include "fl_closed_form.h"
#include "fl_internal.h"
#include "fuselink_hip.h"
#include "fuselink_net.h"

namespace {

// ------------------------------------------------------------------------------------------------
// logging and parameters
// ------------------------------------------------------------------------------------------------
ncclDebugLogger_t g_log = nullptr;
#define FL_WARN(...) do { if (g_log) g_log(NCCL_LOG_WARN, NCCL_ALL, __FILE__, __LINE__, __VA_ARGS__); } while (0)
#define FL_INFO(flags, ...) do { if (g_log) g_log(NCCL_LOG_INFO, (flags), __FILE__, __LINE__, __VA_ARGS__); } while (0)

constexpr int kEngineSetsMax = 8;
struct Params {
  int lanes = 8;                 // virtual NICs = staging lanes (the experiment uses 8 HCAs, run_bw_test.sbatch:43)
  int priority_dev = 0;          // NCCL_FUSELINK_PRIORITY_DEV, plugin.cc:117
  int64_t chunk = 512 << 10;     // NCCL_P2P_NET_CHUNKSIZE of the experiment, run_bw_test.sbatch:34
  int refresh_batch = FL_NET_REFRESH_BATCH;
  int policy = 1;                // 0 = static lane = channelId % lanes (fuselink.h:235); 1 = credit-weighted
  int pool_units = FLH_POOL_UNITS;
  int window_units = 4;          // staging units bound per lane, once per GPU that stages: every connection to that GPU shares the windows
  int qps = 1;                   // NCCL_IB_QPS_PER_CONNECTION, plugin.cc:584
  int split_on_qps = 1;          // NCCL_IB_SPLIT_DATA_ON_QPS, plugin.cc:1410
  int device = -1;               // HIP device that stages; -1 = the one that owns the registered memory
  int idle_credit = 4;
  int max_wave_chunks = 4096;
  int batch = FLH_BATCH_MAX;     // matched sends that may wait for one launch (1 = launch inside isend)
  // How a launch's completion reaches `test`: 0 = an event recorded behind every launch (a barrier packet of its
  // own, some 4.5 us in which the stream's next kernel does not start), 1 = the event rides on the launch's last
  // kernel, 2 = no event and no call into the runtime: pinned words that kernels store launch numbers to
  // (flh_uniform_params).  Every striping kernel, as it starts, stores its launch's number (the launches before it
  // are then complete: a stream runs in order); the reassembly kernel of a launch under 8 MiB also stores the number
  // itself when its last workgroup has finished, after every workgroup's stores have been released, so that a small
  // launch is seen complete without a successor (in a large launch the per-workgroup release costs more than it
  // saves).  A large launch that nothing follows gets an event when it is first polled.
  int completion = 2;
  int small_tile = 0;            // copy tile of a launch under 32 MiB (0 = the library's default tile)
  // NCCL_FUSELINK_ENGINE=1: batches of small requests go to a resident kernel through a descriptor ring instead of
  // through a launch pair each (flh_engine_*); 0 = every batch is a launch pair
  int engine = 1;
  int engine_units = 2;          // staging units per lane for each of the engine's window sets
  int engine_sets = 3;           // window sets the engine's batches rotate through = batches it has in flight at once
  int engine_idle_us = 200;      // the engine goes down after this long without work
  // NCCL_FUSELINK_ENGINE_RESIDENT_US: ... and after this long even with work (0 = never), so that its hardware queue
  // drains; the next batch starts it again.  With eight more streams of the process busy beside the plugin's (more streams
  // than hardware queues), a small fill on one of them waited up to 4.7 ms behind an engine that stayed for as long as
  // requests came (1 GiB in 512 KiB requests, about 5 ms), 2.0 ms with a bound of 2000, 1.0 ms with 1000, 0.8 ms with 500
  // or 250 -- and 0.8 ms with no engine at all.  Every restart costs the transfer a launch: the same 1 GiB moved at
  // 945-990 GB/s with a bound of 1000 or more and at 780-970 with 500 or 250.
  int engine_resident_us = 1000;
  // NCCL_FUSELINK_ONE_PASS: 1 = a launch that can write the receive buffer itself (receiver in this process, or its
  // buffer mapped here) stages and delivers in one kernel, every vector loaded once and stored twice, as the engine's
  // batches do; 0 = a striping launch and a reassembly launch out of the windows
  int one_pass = 1;
  int engine_workgroups = 0;     // 0 = the library's default
  int64_t engine_share1_tiles = -1;   // NCCL_FUSELINK_ENGINE_SHARE1_TILES: flh_tune("lane_share1_tiles"), -1 = the library's default
  int64_t engine_max_request = 1 << 20;   // requests above this size travel by launches
  int queue_depth = 2;           // NCCL_FUSELINK_QUEUE_DEPTH: a test launches what waits while fewer launches than this are queued on the GPU
  // NCCL_FUSELINK_EAGER_BATCH: this many waiting requests are a batch worth its own trip through the engine and go out
  // without a free queue slot, as long as a window set is free (0 = never).  Four connections at NCCL's request shape:
  // 2 000-2 150 GB/s with three sets and 6, against 1 900-1 930 with two sets and the queue depth alone.
  int eager_batch = 6;
  // NCCL_FUSELINK_LIGHT_LOAD: while the engine's batches in flight hold fewer requests than this, what waits goes out
  // past the queue depth as well, as long as a window set is free.  One connection keeps eight requests in flight: its
  // batches of two to three are worth a third slot (850-910 against 740 GB/s); four connections' batches of seven are not.
  int light_load = 8;
  int batch_wait_ns = 2000;      // NCCL_FUSELINK_BATCH_WAIT_NS: a small matched send waits this long for company before a test launches it
  int wire_sets = 4;             // NCCL_FUSELINK_WIRE_SETS: sets of landing windows a receiving process keeps per sending process and GPU = waves on the wire at once
  int wire = 0;                  // NCCL_FUSELINK_WIRE: 0 = both ends in this process (loopback), 1 = the other end is another process (shared-memory wire)
  // NCCL_FUSELINK_WIRE_DIRECT: 1 = a receiver exports the allocations it registers (under 2 GiB) and the sender's second
  // copy writes into the posted buffer itself, as an RDMA write lands in registered memory; 0 = every wave goes through
  // the landing windows and the receiver's own engine or launches deliver it
  int wire_direct = 1;
  int trace = 0;                 // NCCL_FUSELINK_TRACE=1: time spent inside the entry points (fl_net_host_stats)
  int test_early_send = 0;       // NCCL_FUSELINK_TEST_EARLY_SEND=1 under NCCL_FUSELINK_TEST_HOOKS=1: timing experiment, see fl_test
};
Params g_par;

// updateTxChannelActive / updateRxChannelActive (fuselink.h:247-259): every send and every completed receive stamps its
// NIC's entry of the monitor's table, under the table's lock (a semaphore when the table is shared between processes).
// With eight proxy threads at a request every microsecond that lock was the busiest line in the process: each stamp
// cost its caller one to two microseconds.  A NIC's entry is therefore stamped at most once in kMarkEveryUs, a tenth
// of the monitor's timeout (FL_NET_MONITOR_TIMEOUT_US): the table's time of last activity is at most that much older
// than the truth, and a NIC in use can never look idle.
constexpr int64_t kMarkEveryUs = FL_NET_MONITOR_TIMEOUT_US / 10;
alignas(64) std::atomic<int64_t> g_last_mark[2][FL_NET_MAX_LANES];
inline void mark_nic_active(int nic, int is_tx) {
  const int64_t now = fl_monitor_now();
  std::atomic<int64_t>& cell = g_last_mark[is_tx ? 1 : 0][nic];
  int64_t last = cell.load(std::memory_order_relaxed);
  if (last != 0 && now >= last && now - last < kMarkEveryUs) return;
  if (!cell.compare_exchange_strong(last, now, std::memory_order_relaxed)) return;   // another thread stamps it now
  (void)fl_monitor_mark_active(nic, is_tx, now);
}
std::mutex g_init_mu;            // ncclIbLock, plugin.cc:84

// A lock for sections of a few dozen nanoseconds that two proxy threads enter millions of times a second (a
// connection's descriptor ring and counters, the peer's queue of waiting sends).  It spins: a std::mutex puts the loser
// to sleep, and the wake-up costs several microseconds -- with a sender and a receiver thread polling one connection,
// completions that were already visible were seen 7 us late at the median and 19 us late at the 90th percentile.  After
// a few thousand tries it yields, for the case that the holder has lost its core.
class ShortLock {
  std::atomic<bool> held{false};
 public:
  void lock() {
    for (int spins = 0;;) {
      if (!held.exchange(true, std::memory_order_acquire)) return;
      while (held.load(std::memory_order_relaxed)) {
        if (++spins < 4096) {
#if defined(__x86_64__) || defined(__i386__)
          __builtin_ia32_pause();
#endif
        } else {
          std::this_thread::yield();
          spins = 0;
        }
      }
    }
  }
  bool try_lock() { return !held.load(std::memory_order_relaxed) && !held.exchange(true, std::memory_order_acquire); }
  void unlock() { held.store(false, std::memory_order_release); }
};

// NCCL_FUSELINK_TRACE=1: calls and nanoseconds spent inside the entry points and inside the launches they make
// (fl_net_host_stats).  Off, a probe costs one predictable branch.
enum : int { kTrIsend = 0, kTrIrecv, kTrTest, kTrTestDone, kTrFlush, kTrLaunch, kTrRequestsLaunched, kTrEngineSubmit, kTrEngineStart, kTrCount };
// Every thread counts into a block of its own (the blocks live as long as the process; fl_net_host_stats sums them):
// counters shared by eight proxy threads that poll every few hundred nanoseconds cost each probe more than what it measures.
struct TraceCounters { alignas(64) std::atomic<int64_t> calls[kTrCount]; std::atomic<int64_t> ns[kTrCount]; };
std::mutex g_tr_mu;
std::vector<TraceCounters*> g_tr_blocks;
inline void tr_add(int what, int64_t calls, int64_t ns) {
  thread_local TraceCounters* mine = [] {
    TraceCounters* t = new TraceCounters();
    for (int k = 0; k < kTrCount; ++k) { t->calls[k].store(0, std::memory_order_relaxed); t->ns[k].store(0, std::memory_order_relaxed); }
    std::lock_guard<std::mutex> g(g_tr_mu);
    g_tr_blocks.push_back(t);
    return t;
  }();
  // one writer per block: a load and a store, no locked instruction
  mine->calls[what].store(mine->calls[what].load(std::memory_order_relaxed) + calls, std::memory_order_relaxed);
  if (ns) mine->ns[what].store(mine->ns[what].load(std::memory_order_relaxed) + ns, std::memory_order_relaxed);
}
inline int64_t tr_now() {
  timespec t;
  clock_gettime(CLOCK_MONOTONIC, &t);
  return (int64_t)t.tv_sec * 1000000000ll + t.tv_nsec;
}
// NCCL_FUSELINK_TRACE=2 also keeps a timeline: (nanoseconds, thread, event, value) of every entry-point event, in a fixed
// ring that fl_net_timeline() copies out.  Events: 1 irecv posted (value = channel), 2 isend matched (channel),
// 3 pass that launches begins (requests waiting), 4 batch handed over (requests << 32 | number; bit 31 of the number's
// word set for engine batches), 5 request seen complete by test (its batch's number << 16 | bit 15: an engine batch | channel << 1 | is-receive),
// 6 a test call is the first to see the engine's batches complete up to this number, 7 wave announced to the receiving process
// (its number), 8 wave taken off the wire by the receiving process (its number).
struct TimelineEvent { int64_t ns; uint32_t thread; uint32_t event; uint64_t value; };
constexpr size_t kTimelineCap = 1 << 16;
TimelineEvent g_timeline[kTimelineCap];
std::atomic<uint64_t> g_timeline_n{0};
inline void tl_event(uint32_t event, uint64_t value) {
  if (g_par.trace < 2) return;
  static std::atomic<uint32_t> next_thread{0};
  thread_local uint32_t me = next_thread.fetch_add(1);
  const uint64_t i = g_timeline_n.fetch_add(1, std::memory_order_relaxed);
  if (i >= kTimelineCap) return;
  g_timeline[i] = TimelineEvent{tr_now(), me, event, value};
}
struct TraceScope {
  int what;
  int64_t t0;
  explicit TraceScope(int w) : what(w), t0(g_par.trace ? tr_now() : 0) {}
  ~TraceScope() {
    if (!t0) return;
    tr_add(what, 1, tr_now() - t0);
  }
};
bool g_inited = false;

std::mutex g_credit_mu;
bool g_credit_override = false;
uint32_t g_credit_static[FL_NET_MAX_LANES] = {};

std::atomic<int> g_live_links{0};
std::map<int, flh_pool*> g_pools;   // staging units, one pool per HIP device that has registered memory
std::mutex g_pool_mu;

// The calling thread's current device is put back when a plugin call that had to switch it returns: the
// proxy thread that calls in keeps the device its communicator set.
struct DeviceScope {
  int saved = -1;
  DeviceScope() { if (hipGetDevice(&saved) != hipSuccess) saved = -1; }
  ~DeviceScope() { if (saved >= 0) (void)hipSetDevice(saved); }
  DeviceScope(const DeviceScope&) = delete;
  DeviceScope& operator=(const DeviceScope&) = delete;
};
// The same, but the runtime is only asked once a call that needs the device is about to be made: a pass that hands
// everything to the lane engine makes none.
struct LazyDevice {
  int want, saved = -1;
  bool switched = false, ok = true;
  explicit LazyDevice(int device) : want(device) {}
  bool use() {
    if (!switched) {
      switched = true;
      if (hipGetDevice(&saved) != hipSuccess) saved = -1;
      ok = saved == want || hipSetDevice(want) == hipSuccess;
      if (saved == want) saved = -1;   // nothing to put back
    }
    return ok;
  }
  ~LazyDevice() { if (switched && saved >= 0) (void)hipSetDevice(saved); }
  LazyDevice(const LazyDevice&) = delete;
  LazyDevice& operator=(const LazyDevice&) = delete;
};

void parse_credit_env() {
  const char* v = getenv("NCCL_FUSELINK_CREDITS");
  if (!v || !*v) return;
  int n = 0;
  const char* p = v;
  while (*p && n < FL_NET_MAX_LANES) {
    char* end = nullptr;
    long x = strtol(p, &end, 10);
    if (end == p) break;
    g_credit_static[n++] = x < 0 ? 0 : (uint32_t)x;
    p = *end == ',' ? end + 1 : end;
  }
  for (int l = n; l < FL_NET_MAX_LANES; ++l) g_credit_static[l] = 0;
  g_credit_override = n > 0;
}

// ------------------------------------------------------------------------------------------------
// objects
// ------------------------------------------------------------------------------------------------
enum : int { kReqUnused = 0, kReqSend = 1, kReqRecv = 2, kReqFlush = 3 };  // plugin.cc:462-465
enum : int { kStPosted = 1, kStLaunched = 2, kStDoneHost = 3, kStQueued = 4 };

struct Link;
struct WireEnd;
struct WirePair;

struct Request {
  int type = kReqUnused;
  std::atomic<int> state{0};
  Link* link = nullptr;
  uint64_t seq = 0;          // number of the launch (or engine batch) that carries it, counted from 1
  bool engine = false;       // carried by an engine batch, not by a launch
  int size = 0;          // bytes moved (reported by test for receives)
  int fault = 0;         // injected wire fault
  uint32_t magic = 0;
  uint32_t imm = 0xffffffffu;   // receive: the sender's lane-availability mask that came with the data (imm_data, plugin.cc:1463, 1884-1885)
  uint64_t wave = 0;         // send to another process: the wave (of its pair) that must be announced before the send is reported
};
constexpr uint32_t kReqMagic = 0x464c5251;   // "FLRQ"
constexpr uint32_t kCommMagic = 0x464c434d;  // "FLCM"
constexpr uint32_t kMhMagic = 0x464c4d48;    // "FLMH"

// The descriptor a receiver posts: the reference's ncclIbSendFifo (plugin.cc:487-496), 64 bytes, with
// the credit row and an epoch flag carried in what is padding there.
struct FifoWire {
  uint64_t addr;
  int32_t size;
  uint32_t rkey;
  uint32_t nreqs;
  uint32_t tag;
  uint64_t idx;
  int32_t fuselink_offset;   // >= 0: the whole request goes to this lane; -1: comm's own lane; -2: credit row below
  uint8_t credits[FL_NET_MAX_LANES];
  uint32_t flags;            // bit 0: the receiver refreshed its lane decision (new credit epoch)
  uint8_t pad[8];
};
static_assert(sizeof(FifoWire) == 64, "descriptor must stay one 64-byte slot");

struct FifoSlot {
  FifoWire w;
  Request* rreq;     // loopback only: the receive request this descriptor belongs to
  int rtype;         // pointer type of the receive buffer
  int rdevice;       // HIP device of the receive buffer (-1: host memory)
};

// a matched send whose GPU work has not been queued yet
struct Pending {
  Link* lk;
  const uint8_t* src;
  uint8_t* dst;
  int size;
  bool src_dev, dst_dev;
  FifoWire w;
  Request *sreq, *rreq;      // (rreq: null when the receiver is another process)
  uint32_t imm = 0xffffffffu;   // the sender's lane-availability mask that travels with the request
  uint64_t fifo_idx = 0;     // the descriptor it answers, from 1
  int q_next = 0;            // a send to another process that travels wave by wave: the QP piece it has got to ...
  uint64_t q_done = 0;       // ... and the bytes of that piece that are on their way
  bool direct = false;       // a send to another process whose posted buffer this process can write itself (dst is that mapping)
};

// What one launch pair carried, for inspection (fl_net_last_launch).
struct LaunchSeg {
  int channelId;
  uint32_t first_row, n_rows, n_req;
  uint64_t epoch_bytes;
  uint64_t lane_base[FL_NET_MAX_LANES];
};
struct LaunchInfo {
  bool engine = false;       // an engine batch: its table sits in the engine's slot (seq - 1) % kEngineSlots
  uint64_t seq = 0;
  uint32_t n_seg = 0, n_rows = 0;
  LaunchSeg seg[FLH_SEG_MAX] = {};
};

constexpr size_t kEventRing = 1024;

// The staging side of one GPU, shared by every connection that stages there, as the reference's per-NIC lane comms
// are shared by all channels (fuselink.h:271-272; opened once, on the first connect, plugin.cc:727-753): one stream,
// one staging window per lane, one queue of matched sends, one sequence of launch numbers.
constexpr uint32_t kEngineSlots = 64;              // the engine's descriptor ring
constexpr uint32_t kEngineRows = 512;              // chunks an engine batch may hold
struct Peer {
  int hip_device = 0;
  int links = 0;                    // connections attached (g_peer_mu)
  bool ready = false;
  hipStream_t stream = nullptr;
  flh_window* win[FL_NET_MAX_LANES] = {};
  flh_windows wins = {};
  flh_chunk_desc* d_table = nullptr;
  flh_sched_hdr* d_hdr = nullptr;
  uint32_t* d_count = nullptr;      // device word in which a reassembly launch counts its finished workgroups
  int32_t* h_status = nullptr;      // pinned, device-visible: kernels report range refusals here
  int32_t* d_status = nullptr;
  uint32_t* h_done = nullptr;       // pinned, device-visible: number of the last launch whose reassembly kernel reported itself finished (completion mode 2)
  uint32_t* d_done = nullptr;
  uint32_t* h_started = nullptr;    // pinned, device-visible: number of the last launch whose striping kernel has started
  uint32_t* d_started = nullptr;
  // matched sends that wait for a launch, in arrival order.  (Cache lines: what the senders write, what the pollers
  // read and what only the thread that launches touches are kept apart; polling threads must not slow a launch down by
  // pulling its lines away.)
  alignas(64) ShortLock queue_mu;
  std::vector<Pending> pending;
  std::atomic<uint32_t> waiting_reqs{0};
  std::atomic<uint64_t> waiting_bytes{0};
  std::atomic<int64_t> waiting_since{0};   // monotonic nanoseconds at which the oldest waiting send arrived
  // Guards every launch on `stream`, the event ring, the launch numbers, the connections' scheduling state
  // (epoch_bytes, launch counters, last table) and `last`.  Taken before queue_mu, never the other way round.
  alignas(64) std::mutex launch_mu;
  alignas(64) std::atomic<bool> launching{false};   // a thread holds launch_mu for a pass: pollers look here before they try the lock
  alignas(64) std::vector<Pending> work;        // the waiting sends a flush took over (launch_mu)
  std::vector<Pending> work_sorted; // scratch of the same pass
  std::vector<bool> work_taken;
  hipEvent_t evring[kEventRing] = {};              // launch n may own slot (n - 1) % kEventRing
  std::atomic<uint64_t> ev_seq[kEventRing] = {};   // the launch whose completion the slot's event stands for (0: none)
  alignas(64) std::atomic<uint64_t> done_seq{0};   // highest launch number known complete; launches run in order on one stream
  std::atomic<uint64_t> launch_seq{0};             // highest launch number handed out
  std::atomic<uint64_t> last_event_seq{0};         // highest launch whose completion comes from an event, not from the word
  alignas(64) LaunchInfo last;
  // the lane engine (flh_engine_*): a resident kernel that takes batches of small requests from a descriptor ring.
  // Its batches alternate between two window sets of their own and have their own numbers, tables and headers.
  flh_engine* engine = nullptr;
  std::atomic<bool> engine_ok{false};              // cleared for good when the engine reports an error
  std::atomic<uint64_t> tl_engine_seen{0};         // timeline only: the engine batches some test call has seen complete
  flh_window* ewin[kEngineSetsMax][FL_NET_MAX_LANES] = {};
  flh_windows ewins[kEngineSetsMax] = {};
  int engine_sets = 0;             // window sets that were bound (NCCL_FUSELINK_ENGINE_SETS, or as many as the pool held)
  flh_chunk_desc* d_etable = nullptr;              // kEngineSlots tables of kEngineRows rows
  flh_sched_hdr* d_ehdr = nullptr;                 // kEngineSlots headers
  alignas(64) std::atomic<uint64_t> engine_submitted{0};   // batches handed to the engine (written under launch_mu)
  std::atomic<uint64_t> engine_reqs_upto[kEngineSlots] = {};   // requests in batches 1..k, at k mod the ring: what the engine holds is a difference of two
};

struct Link {
  ShortLock mu;
  int refs = 2;                     // one per side
  int dev = 0;                      // NIC index the comms were opened on
  int channelId = 0;                // plugin.cc:693-708
  int send_ready = 0;               // comm->ready, plugin.cc:1502; -1: the listener closed before accepting
  // sender side
  FifoSlot fifo[FL_NET_MAX_REQUESTS];
  uint64_t fifoHead = 0;            // plugin.cc:1510
  Request sreq[FL_NET_MAX_REQUESTS];
  int64_t s_finished = 0, s_inflight = 0;
  // receiver side
  uint64_t fifoTail = 0;            // plugin.cc:1619
  Request rreq[FL_NET_MAX_REQUESTS];
  int64_t r_finished = 0, r_inflight = 0, refreshes = 0;
  int fuselink_offset = -1;
  uint8_t credits[FL_NET_MAX_LANES] = {};
  bool have_decision = false;
  // The sender's lane-availability mask (getTxUsage / refreshTxUsage, fuselink.h:261-267): refreshed every
  // N_FINISHED_BATCH sends (plugin.cc:1441-1447), shipped with every request as its immediate data (plugin.cc:1463).
  uint32_t tx_mask = 0xffffffffu;   // sender: the cached mask (the reference's placeholder value until the first refresh)
  int64_t tx_refreshes = 0;
  uint32_t tx_available = 0xffffffffu;   // receiver: the mask of the latest completed receive (comm->txAvailable, plugin.cc:1884-1885)
  // the other end is another process (NCCL_FUSELINK_WIRE=shm): this end of the shared-memory wire; null on the loopback
  WireEnd* wire = nullptr;
  // staging side: the GPU's shared one, attached on first use with device memory (set once, under mu)
  std::atomic<Peer*> peer{nullptr};
  // scheduling state of the connection (the peer's launch_mu)
  uint64_t epoch_bytes = 0;         // bytes scheduled since the last lane-decision refresh (the scheduler's carried prefix)
  uint64_t last_seq = 0;            // launch that carried the connection's latest segment, and that segment's rows in its table
  bool last_engine = false;         // ... or engine batch
  uint32_t last_first_row = 0, last_rows = 0;
  int64_t launches = 0, batched_requests = 0;    // launch pairs that carried its requests, requests that shared a pair with others
};

struct Comm {
  uint32_t magic = kCommMagic;
  int is_send = 0;
  Link* link = nullptr;
};

struct ListenComm {
  uint32_t magic = kCommMagic;
  int dev = 0;
  int channelId = 0;
  uint64_t id = 0;
  std::deque<Link*> pending;   // connects waiting for accept
};

struct MemHandle {             // FuseLinkMemHandle, fuselink.h:48-52
  uint32_t magic = kMhMagic;
  int type = 0;
  uintptr_t start_addr = 0;
  size_t size = 0;
  flh_region* region = nullptr;  // shared per base allocation (device memory only)
  int device = -1;               // HIP device that owns the memory (-1: host memory)
  // registered on a receiving comm whose sender is another process: the key under which that process may write into
  // the allocation directly (0: it cannot), and the pair of processes the key belongs to
  WirePair* wire_pair = nullptr;
  uint32_t rkey = 0;
  // registered through regMrDmaBuf with a descriptor: this registration's own duplicate of it and the offset that came
  // with it (what the reference hands to ibv_reg_dmabuf_mr for every relay buffer, plugin.cc:1278-1280), kept for a
  // wire that registers memory with a NIC; closed when the registration goes
  int dmabuf_fd = -1;
  uint64_t dmabuf_offset = 0;
  ~MemHandle() { if (dmabuf_fd >= 0) close(dmabuf_fd); }
};

struct Handle {                // what listen writes into the caller's 128 bytes (plugin.cc:425-430)
  uint64_t magic;
  uint64_t listen_id;
  int32_t channelId;
  int32_t dev;
  int32_t stage;               // 0 start, 1 connect posted (plugin.cc:407-423)
  int32_t pad;
  void* stage_link;
};
static_assert(sizeof(Handle) < NCCL_NET_HANDLE_MAXSIZE, "handle must fit the caller's buffer");  // plugin.cc:705
constexpr uint64_t kHandleMagic = 0x4655534c494e4b31ull;

std::mutex g_reg_mu;                        // listen registry + channel counter (plugin.cc:690-698)
std::map<uint64_t, ListenComm*> g_listens;
uint64_t g_next_listen = 1;
int g_channel_counter = 0;

ncclResult_t hip_fail(const char* what, hipError_t e) {
  FL_WARN("NET/FuseLink : %s failed: %s", what, hipGetErrorString(e));
  return ncclUnhandledCudaError;   // where the reference exit(1)s (src/checks.h:17-23)
}
#define FL_HIPCHECK(call) do { hipError_t e_ = (call); if (e_ != hipSuccess) return hip_fail(#call, e_); } while (0)
#define FL_FLHCHECK(call) do { int rc_ = (call); if (rc_ < 0) { FL_WARN("NET/FuseLink : %s: %s", #call, flh_last_error()); \
  return rc_ == FLH_E_NOMEM || rc_ == FLH_E_ARG ? ncclInternalError : ncclUnhandledCudaError; } } while (0)

std::mutex g_peer_mu;                // the peers, their attachment counts
std::map<int, Peer*> g_peers;        // one per HIP device that stages

void flush_pending(Peer* pr);
void wire_end_free(Link* lk);

void peer_destroy(Peer* pr) {        // no longer reachable through g_peers
  DeviceScope keep;
  (void)hipSetDevice(pr->hip_device);
  if (pr->engine) (void)flh_engine_destroy(pr->engine);   // asks the resident kernel down and waits for it
  if (pr->stream) (void)hipStreamSynchronize(pr->stream);
  for (int l = 0; l < FL_NET_MAX_LANES; ++l) {
    if (pr->win[l]) (void)flh_window_destroy(pr->win[l]);
    for (int h = 0; h < kEngineSetsMax; ++h) if (pr->ewin[h][l]) (void)flh_window_destroy(pr->ewin[h][l]);
  }
  if (pr->d_etable) (void)hipFree(pr->d_etable);
  if (pr->d_ehdr) (void)hipFree(pr->d_ehdr);
  if (pr->d_table) (void)hipFree(pr->d_table);
  if (pr->d_hdr) (void)hipFree(pr->d_hdr);
  if (pr->d_count) (void)hipFree(pr->d_count);
  if (pr->h_status) (void)hipHostFree(pr->h_status);
  for (auto& e : pr->evring) if (e) (void)hipEventDestroy(e);
  if (pr->stream) (void)hipStreamDestroy(pr->stream);
  delete pr;
}

void link_unref(Link* lk) {
  bool last;
  {
    std::lock_guard<ShortLock> g(lk->mu);
    last = --lk->refs == 0;
  }
  if (!last) return;
  Peer* const peer = lk->peer.load(std::memory_order_acquire);
  if (peer) {   // nothing of this connection may still wait for a launch when it goes away
    std::lock_guard<std::mutex> g(peer->launch_mu);
    flush_pending(peer);
    // (sends to another process that found no landing set free stay queued: they go with their connection)
    std::lock_guard<ShortLock> gq(peer->queue_mu);
    size_t kept = 0;
    for (size_t i = 0; i < peer->pending.size(); ++i) {
      if (peer->pending[i].lk == lk) continue;
      if (kept != i) peer->pending[kept] = peer->pending[i];
      ++kept;
    }
    if (kept != peer->pending.size()) {
      peer->pending.resize(kept);
      uint64_t bytes = 0;
      for (const Pending& q : peer->pending) bytes += (uint64_t)q.size;
      peer->waiting_reqs.store((uint32_t)kept, std::memory_order_release);
      peer->waiting_bytes.store(bytes, std::memory_order_release);
    }
  }
  wire_end_free(lk);   // (before the staging side: a receiver's landing windows wait for its stream)
  if (Peer* pr = peer) {
    bool gone;
    {
      std::lock_guard<std::mutex> g(g_peer_mu);
      gone = --pr->links == 0;
      if (gone) g_peers.erase(pr->hip_device);
    }
    if (gone) peer_destroy(pr);   // the last connection that staged on this GPU: windows and stream go back
  }
  delete lk;
  g_live_links.fetch_sub(1);
}

// first free of 256 (ncclIbGetRequest, plugin.cc:1070-1085)
Request* get_request(Request* tab, Link* lk, int type) {
  for (int i = 0; i < FL_NET_MAX_REQUESTS; ++i) {
    Request* r = tab + i;
    if (r->type == kReqUnused) {
      r->type = type;
      r->link = lk;
      r->size = 0;
      r->seq = 0;
      r->engine = false;
      r->fault = 0;
      r->magic = kReqMagic;
      r->state.store(0, std::memory_order_relaxed);
      return r;
    }
  }
  FL_WARN("NET/FuseLink : unable to allocate requests");
  return nullptr;
}

// The pool of the device (created on first use; creating it makes that device current).
ncclResult_t ensure_pool(int device, flh_pool** out) {
  std::lock_guard<std::mutex> g(g_pool_mu);
  auto it = g_pools.find(device);
  if (it == g_pools.end()) {
    flh_pool* p = nullptr;
    FL_FLHCHECK(flh_pool_create(device, (uint32_t)g_par.pool_units, &p));
    it = g_pools.emplace(device, p).first;
  }
  *out = it->second;
  return ncclSuccess;
}

// Stream, one bound window per lane, table / header buffers, status and completion words of a new peer.
ncclResult_t peer_setup(Peer* pr, int device) {
  flh_pool* pool = nullptr;
  ncclResult_t rc = ensure_pool(device, &pool);
  if (rc != ncclSuccess) return rc;
  pr->hip_device = device;
  FL_HIPCHECK(hipSetDevice(device));
  FL_HIPCHECK(hipStreamCreateWithFlags(&pr->stream, hipStreamNonBlocking));
  const uint64_t cap = (uint64_t)g_par.window_units * FLH_UNIT_BYTES;
  memset(&pr->wins, 0, sizeof(pr->wins));
  pr->wins.n_lanes = (uint32_t)g_par.lanes;
  for (int l = 0; l < g_par.lanes; ++l) {
    FL_FLHCHECK(flh_window_create(pool, cap, &pr->win[l]));
    FL_FLHCHECK(flh_window_bind(pr->win[l], cap));
    pr->wins.base[l] = flh_window_base(pr->win[l]);
    pr->wins.cap[l] = flh_window_bound_bytes(pr->win[l]);
  }
  FL_HIPCHECK(hipMalloc((void**)&pr->d_table, sizeof(flh_chunk_desc) * (size_t)g_par.max_wave_chunks));
  FL_HIPCHECK(hipMalloc((void**)&pr->d_hdr, sizeof(flh_sched_hdr)));
  FL_HIPCHECK(hipMalloc((void**)&pr->d_count, 256));
  FL_HIPCHECK(hipMemset(pr->d_count, 0, 256));
  FL_HIPCHECK(hipHostMalloc((void**)&pr->h_status, 256, hipHostMallocMapped));   // status word and the two completion words, a cache line apart
  memset(pr->h_status, 0, 256);
  FL_HIPCHECK(hipHostGetDevicePointer((void**)&pr->d_status, pr->h_status, 0));
  pr->h_done = (uint32_t*)((char*)pr->h_status + 64);
  pr->d_done = (uint32_t*)((char*)pr->d_status + 64);
  pr->h_started = (uint32_t*)((char*)pr->h_status + 128);
  pr->d_started = (uint32_t*)((char*)pr->d_status + 128);
  if (g_par.engine) {
    const uint64_t ecap = (uint64_t)g_par.engine_units * FLH_UNIT_BYTES;
    if (ecap < (uint64_t)g_par.chunk) {
      FL_INFO(NCCL_NET, "NET/FuseLink : the engine's windows (%llu bytes) do not hold a chunk: launches only", (unsigned long long)ecap);
    } else {
      // as many window sets as asked for, or as the pool still holds whole: the launches' windows come first
      int sets = 0;
      for (int h = 0; h < g_par.engine_sets; ++h) {
        bool whole = true;
        for (int l = 0; l < g_par.lanes && whole; ++l)
          whole = flh_window_create(pool, ecap, &pr->ewin[h][l]) >= 0 && flh_window_bind(pr->ewin[h][l], ecap) >= 0;
        if (!whole) {
          for (int l = 0; l < g_par.lanes; ++l)
            if (pr->ewin[h][l]) { (void)flh_window_destroy(pr->ewin[h][l]); pr->ewin[h][l] = nullptr; }
          break;
        }
        pr->ewins[h].n_lanes = (uint32_t)g_par.lanes;
        for (int l = 0; l < g_par.lanes; ++l) {
          pr->ewins[h].base[l] = flh_window_base(pr->ewin[h][l]);
          pr->ewins[h].cap[l] = flh_window_bound_bytes(pr->ewin[h][l]);
        }
        ++sets;
      }
      if (sets == 0) {
        FL_INFO(NCCL_NET, "NET/FuseLink : the pool has no room for a window set of the engine: launches only");
      } else {
        if (sets < g_par.engine_sets) FL_INFO(NCCL_NET, "NET/FuseLink : the pool holds %d of the engine's %d window sets", sets, g_par.engine_sets);
        pr->engine_sets = sets;
        FL_HIPCHECK(hipMalloc((void**)&pr->d_etable, sizeof(flh_chunk_desc) * (size_t)kEngineSlots * kEngineRows));
        FL_HIPCHECK(hipMalloc((void**)&pr->d_ehdr, sizeof(flh_sched_hdr) * (size_t)kEngineSlots));
        FL_FLHCHECK(flh_engine_create(device, (uint32_t)g_par.engine_workgroups, (uint32_t)g_par.engine_idle_us, (uint32_t)sets, &pr->engine));
        FL_FLHCHECK(flh_engine_set_resident(pr->engine, (uint32_t)g_par.engine_resident_us));
        pr->engine_ok.store(true, std::memory_order_release);
      }
    }
  }
  pr->ready = true;
  FL_INFO(NCCL_NET, "NET/FuseLink : device %d staging ready: %d lanes x %llu bytes, shared by its connections", device, g_par.lanes, (unsigned long long)cap);
  return ncclSuccess;
}

// Attach the connection to the staging side of `device`, which owns the buffer that is being registered or sent
// (lk->mu held).  The connection stages there from then on.
ncclResult_t attach_peer(Link* lk, int device) {
  if (lk->peer.load(std::memory_order_acquire)) return ncclSuccess;
  if (device < 0) { FL_WARN("NET/FuseLink : no HIP device to stage on"); return ncclInternalError; }
  DeviceScope keep;
  std::lock_guard<std::mutex> g(g_peer_mu);
  auto it = g_peers.find(device);
  if (it == g_peers.end()) {
    Peer* pr = new (std::nothrow) Peer();
    if (!pr) return ncclSystemError;
    ncclResult_t rc = peer_setup(pr, device);
    if (rc != ncclSuccess) { peer_destroy(pr); return rc; }
    it = g_peers.emplace(device, pr).first;
  }
  it->second->links++;
  lk->peer.store(it->second, std::memory_order_release);
  return ncclSuccess;
}

// Credit row the receiver advertises at a refresh: refreshRxComm(channelId, txAvailable, ...) of plugin.cc:1710 with the
// query the reference left commented out (fuselink.h:240-243, getIdleNicRx(group, priority, txAvailable)) -- a lane
// counts when its receive side is idle in this host's table and the sender's mask admits it.  tx_available is the mask
// that came with the latest completed receive.  Both ends in one process read one table: there the receiver reads the
// send statuses themselves, as they are now, in place of the sender's last report of them (which is up to a batch old).
void current_credits(int own_lane, uint32_t tx_available, bool same_process, uint8_t* out) {
  uint32_t c[FL_NET_MAX_LANES] = {};
  {
    std::lock_guard<std::mutex> g(g_credit_mu);
    if (g_credit_override) {
      for (int l = 0; l < g_par.lanes; ++l) c[l] = g_credit_static[l];
    } else {
      // the daemon's periodic ageing (monitor.cpp:159-193) happens here, right before the table is read
      (void)fl_monitor_tick(fl_monitor_now());
      uint32_t mask = tx_available;
      if (same_process) (void)fl_monitor_tx_mask(g_par.lanes, own_lane, &mask);
      (void)fl_monitor_rx_credits(g_par.lanes, own_lane, (uint32_t)g_par.idle_credit, mask, c);
    }
  }
  for (int l = 0; l < FL_NET_MAX_LANES; ++l) out[l] = (uint8_t)(c[l] > 255 ? 255 : c[l]);
}

// The mask a sender ships with a request: cached, refreshed when (n_finished + 1) % N_FINISHED_BATCH == 0
// (plugin.cc:1441-1447; refreshTxUsage / getTxUsage, fuselink.h:261-267, placeholders there).  lk->mu held.
uint32_t sender_mask(Link* lk) {
  if ((lk->s_finished + 1) % g_par.refresh_batch == 0) {
    uint32_t mask = 0xffffffffu;
    bool forced;
    {
      std::lock_guard<std::mutex> g(g_credit_mu);
      forced = g_credit_override;
    }
    if (!forced && g_par.policy != 0) {
      (void)fl_monitor_tick(fl_monitor_now());
      (void)fl_monitor_tx_mask(g_par.lanes, lk->dev % g_par.lanes, &mask);
    }
    lk->tx_mask = mask;
    lk->tx_refreshes++;
  }
  return lk->tx_mask;
}

// Chunks one wave may carry so that no lane outgrows its window: the largest n for which every lane's share
// of the quanta [before, before + n) -- the scheduler's closed form, (x / W) c + clamp(x mod W - K, 0, c) slots
// before quantum x for a lane with first slot K and credit c -- still fits.  A bound that holds for any phase,
// (ceil(n / W) + 1) c chunks for a lane of credit c, is where the search starts.
uint32_t wave_chunks(const uint32_t* credits, int lanes, uint64_t chunk, uint64_t cap, uint64_t quanta_before) {
  uint64_t c[FL_NET_MAX_LANES], K[FL_NET_MAX_LANES], W = 0, cmax = 0;
  for (int l = 0; l < lanes; ++l) W += credits[l];
  for (int l = 0; l < lanes; ++l) c[l] = W ? credits[l] : 1;   // no credit anywhere: equal credits stand in
  W = 0;
  for (int l = 0; l < lanes; ++l) { K[l] = W; W += c[l]; if (c[l] > cmax) cmax = c[l]; }
  const uint64_t per_lane = cap / chunk;           // chunks a window holds
  if (per_lane == 0) return 0;
  const uint64_t rounds = per_lane / cmax;         // (ceil(n / W) + 1) <= rounds
  uint64_t lo = rounds >= 2 ? (rounds - 1) * W : 1;
  uint64_t hi = per_lane * (uint64_t)lanes;        // all windows full
  if (hi > (uint64_t)g_par.max_wave_chunks) hi = (uint64_t)g_par.max_wave_chunks;
  if (lo > hi) lo = hi;
  auto before = [&](int l, uint64_t x) {
    const uint64_t rem = x % W;
    return (x / W) * c[l] + (rem <= K[l] ? 0 : (rem - K[l] < c[l] ? rem - K[l] : c[l]));
  };
  auto fits = [&](uint64_t n) {
    for (int l = 0; l < lanes; ++l)
      if (before(l, quanta_before + n) - before(l, quanta_before) > per_lane) return false;
    return true;
  };
  while (lo < hi) {                                // largest n in [lo, hi] that fits; the shares only grow with n
    const uint64_t mid = lo + (hi - lo + 1) / 2;
    if (fits(mid)) lo = mid; else hi = mid - 1;
  }
  return (uint32_t)lo;
}

// ------------------------------------------------------------------------------------------------
// shared-memory wire: sender and receiver in different processes (NCCL_FUSELINK_WIRE=shm)
// ------------------------------------------------------------------------------------------------
#include "fl_plugin_shm_wire.h"

// ------------------------------------------------------------------------------------------------
// plugin entry points (v8 signatures; v7 / v6 adapt)
// ------------------------------------------------------------------------------------------------
ncclResult_t fl_init(ncclDebugLogger_t logFunction) {
  std::lock_guard<std::mutex> g(g_init_mu);
  g_log = logFunction;
  if (g_inited) return ncclSuccess;
  g_par.lanes = (int)fl_param("FUSELINK_LANES", g_par.lanes);
  g_par.priority_dev = (int)fl_param("FUSELINK_PRIORITY_DEV", g_par.priority_dev);
  g_par.chunk = fl_param("FUSELINK_CHUNKSIZE", g_par.chunk);
  g_par.refresh_batch = (int)fl_param("FUSELINK_REFRESH_BATCH", g_par.refresh_batch);
  g_par.policy = (int)fl_param("FUSELINK_POLICY", g_par.policy);
  g_par.pool_units = (int)fl_param("FUSELINK_POOL_UNITS", g_par.pool_units);
  g_par.window_units = (int)fl_param("FUSELINK_WINDOW_UNITS", g_par.window_units);
  g_par.qps = (int)fl_param("IB_QPS_PER_CONNECTION", g_par.qps);
  g_par.split_on_qps = (int)fl_param("IB_SPLIT_DATA_ON_QPS", g_par.split_on_qps);
  g_par.device = (int)fl_param("FUSELINK_DEVICE", g_par.device);
  g_par.idle_credit = (int)fl_param("FUSELINK_IDLE_CREDIT", g_par.idle_credit);
  g_par.max_wave_chunks = (int)fl_param("FUSELINK_MAX_WAVE_CHUNKS", g_par.max_wave_chunks);
  g_par.batch = (int)fl_param("FUSELINK_BATCH", g_par.batch);
  g_par.completion = (int)fl_param("FUSELINK_COMPLETION", g_par.completion);
  g_par.small_tile = (int)fl_param("FUSELINK_SMALL_TILE", g_par.small_tile);
  if (g_par.small_tile < 0 || g_par.small_tile % 128) { FL_WARN("NET/FuseLink : NCCL_FUSELINK_SMALL_TILE must be a multiple of 128"); return ncclInvalidArgument; }
  g_par.trace = (int)fl_param("FUSELINK_TRACE", g_par.trace);
  {
    const char* hooks = getenv("NCCL_FUSELINK_TEST_HOOKS");
    g_par.test_early_send = hooks && !strcmp(hooks, "1") && fl_param("FUSELINK_TEST_EARLY_SEND", 0) != 0;
  }
  {
    const char* wv = getenv("NCCL_FUSELINK_WIRE");
    g_par.wire = wv && (!strcmp(wv, "shm") || !strcmp(wv, "1")) ? 1 : 0;
  }
  g_par.wire_sets = (int)fl_param("FUSELINK_WIRE_SETS", g_par.wire_sets);
  g_par.wire_direct = (int)fl_param("FUSELINK_WIRE_DIRECT", g_par.wire_direct) != 0;
  if (g_par.wire_sets < 1) g_par.wire_sets = 1;
  if (g_par.wire_sets > kShmSetsMax) g_par.wire_sets = kShmSetsMax;
  g_par.engine = (int)fl_param("FUSELINK_ENGINE", g_par.engine);
  g_par.engine_units = (int)fl_param("FUSELINK_ENGINE_UNITS", g_par.engine_units);
  g_par.engine_idle_us = (int)fl_param("FUSELINK_ENGINE_IDLE_US", g_par.engine_idle_us);
  g_par.engine_resident_us = (int)fl_param("FUSELINK_ENGINE_RESIDENT_US", g_par.engine_resident_us);
  if (g_par.engine_resident_us < 0) g_par.engine_resident_us = 0;
  g_par.engine_sets = (int)fl_param("FUSELINK_ENGINE_SETS", g_par.engine_sets);
  if (g_par.engine_sets < 1 || g_par.engine_sets > kEngineSetsMax) { FL_WARN("NET/FuseLink : NCCL_FUSELINK_ENGINE_SETS must be 1..%d", kEngineSetsMax); return ncclInvalidArgument; }
  g_par.one_pass = (int)fl_param("FUSELINK_ONE_PASS", g_par.one_pass) != 0;
  (void)flh_tune("stream_mode_deliver", fl_param("FUSELINK_DELIVER_STREAM_MODE", -1));   // an experiment's knob: see flh_tune
  g_par.engine_workgroups = (int)fl_param("FUSELINK_ENGINE_WORKGROUPS", g_par.engine_workgroups);
  g_par.engine_share1_tiles = fl_param("FUSELINK_ENGINE_SHARE1_TILES", g_par.engine_share1_tiles);
  (void)flh_tune("lane_share1_tiles", g_par.engine_share1_tiles);
  g_par.engine_max_request = fl_param("FUSELINK_ENGINE_MAX_REQUEST", g_par.engine_max_request);
  if (g_par.engine_units < 1 || g_par.engine_idle_us < 1 || g_par.engine_workgroups < 0) { FL_WARN("NET/FuseLink : engine parameter out of range"); return ncclInvalidArgument; }
  g_par.batch_wait_ns = (int)fl_param("FUSELINK_BATCH_WAIT_NS", g_par.batch_wait_ns);
  if (g_par.batch_wait_ns < 0) g_par.batch_wait_ns = 0;
  g_par.queue_depth = (int)fl_param("FUSELINK_QUEUE_DEPTH", g_par.queue_depth);
  g_par.eager_batch = (int)fl_param("FUSELINK_EAGER_BATCH", g_par.eager_batch);
  g_par.light_load = (int)fl_param("FUSELINK_LIGHT_LOAD", g_par.light_load);
  if (g_par.queue_depth < 1) g_par.queue_depth = 1;
  if (g_par.completion < 0 || g_par.completion > 2) g_par.completion = 2;
  if (g_par.max_wave_chunks > 65535) g_par.max_wave_chunks = 65535;   // what one fused launch can name
  if (g_par.batch < 1) g_par.batch = 1;
  if (g_par.batch > FLH_BATCH_MAX) g_par.batch = FLH_BATCH_MAX;
  if (g_par.completion != 2 || g_par.batch < 2) g_par.engine = 0;   // the engine reports through its completion word and takes batches
  if (g_par.lanes < 1 || g_par.lanes > FL_NET_MAX_LANES) { FL_WARN("NET/FuseLink : NCCL_FUSELINK_LANES must be 1..%d", FL_NET_MAX_LANES); return ncclInvalidArgument; }
  if (g_par.chunk < 128 || g_par.chunk % 128 || g_par.chunk > (int64_t)1 << 30) { FL_WARN("NET/FuseLink : NCCL_FUSELINK_CHUNKSIZE must be a multiple of 128 up to 1 GiB"); return ncclInvalidArgument; }
  if (g_par.refresh_batch < 1 || g_par.qps < 1 || g_par.qps > 128 || g_par.window_units < 1 || g_par.pool_units < 1 || g_par.max_wave_chunks < 1) {
    FL_WARN("NET/FuseLink : parameter out of range");
    return ncclInvalidArgument;
  }
  if ((int64_t)g_par.window_units * FLH_UNIT_BYTES < g_par.chunk) { FL_WARN("NET/FuseLink : a staging window must hold at least one chunk"); return ncclInvalidArgument; }
  parse_credit_env();
  if (fl_param("FUSELINK_MONITOR_SHM", 0)) {
    // lane statuses come from the daemon's shared table, as in FuseLinkConnManager::SetUpMonitor (fuselink.h:99-101);
    // an absent daemon is an error here instead of the exception MonitorClient throws (monitor.h:113-131)
    if (fl_monitor_attach_shm(nullptr, nullptr, 0) != 0) { FL_WARN("NET/FuseLink : %s", flh_last_error()); return ncclSystemError; }
  }
  g_inited = true;
  FL_INFO(NCCL_INIT | NCCL_NET, "NET/FuseLink : %d lanes, chunk %lld, policy %s, refresh every %d requests (loopback wire)", g_par.lanes,
          (long long)g_par.chunk, g_par.policy ? "credits" : "static", g_par.refresh_batch);
  return ncclSuccess;
}

ncclResult_t fl_devices(int* ndev) {
  if (!ndev) return ncclInvalidArgument;
  *ndev = g_par.lanes;  // one virtual NIC per staging lane
  return ncclSuccess;
}

char g_dev_names[FL_NET_MAX_LANES][32];

ncclResult_t fl_get_properties_v8(int dev, ncclNetProperties_v8_t* props) {
  if (!props || dev < 0 || dev >= g_par.lanes) return ncclInvalidArgument;
  snprintf(g_dev_names[dev], sizeof(g_dev_names[dev]), "fuselink%d", dev);
  props->name = g_dev_names[dev];
  props->pciPath = nullptr;
  props->guid = (uint64_t)dev;
  props->ptrSupport = NCCL_PTR_HOST | NCCL_PTR_CUDA | NCCL_PTR_DMABUF;   // plugin.cc:364-370; regMrDmaBuf checks and keeps the descriptor
  props->regIsGlobal = 1;                              // registrations are keyed by base address, not by comm
  props->speed = 400000;
  props->port = 1;
  props->latency = 0;                                  // plugin.cc:372
  props->maxComms = 65536;
  props->maxRecvs = 1;   // the reference advertises 8 (plugin.cc:375) yet rejects grouped receives (plugin.cc:1448-1451)
  props->netDeviceType = NCCL_NET_DEVICE_HOST;         // plugin.cc:376-377
  props->netDeviceVersion = NCCL_NET_DEVICE_INVALID_VERSION;
  return ncclSuccess;
}

ncclResult_t fl_listen(int dev, void* opaqueHandle, void** listenComm) {
  if (!opaqueHandle || !listenComm || dev < 0 || dev >= g_par.lanes) return ncclInvalidArgument;
  if (g_par.wire == 1) return shm_listen(dev, opaqueHandle, listenComm);
  ListenComm* lc = new (std::nothrow) ListenComm();
  if (!lc) return ncclSystemError;
  Handle* h = (Handle*)opaqueHandle;
  memset(h, 0, sizeof(Handle));
  {
    std::lock_guard<std::mutex> g(g_reg_mu);
    lc->id = g_next_listen++;
    lc->channelId = g_channel_counter++;  // ncclIbAllocateChannel, plugin.cc:693-698
    lc->dev = dev;
    g_listens[lc->id] = lc;
  }
  h->magic = kHandleMagic;
  h->listen_id = lc->id;
  h->channelId = lc->channelId;
  h->dev = dev;
  *listenComm = lc;
  FL_INFO(NCCL_INIT | NCCL_NET, "NET/FuseLink : channel id %d listen comm %p dev %d", lc->channelId, (void*)lc, dev);
  return ncclSuccess;
}

// Non-blocking, staged like the reference (plugin.cc:407-423, 721-760): the first call posts the
// connection to the listener and returns NULL; a later call returns the comm once accept() took it.
ncclResult_t fl_connect(int dev, void* opaqueHandle, void** sendComm, ncclNetDeviceHandle_v8_t** /*sendDevComm*/) {
  if (!opaqueHandle || !sendComm || dev < 0 || dev >= g_par.lanes) return ncclInvalidArgument;
  Handle* h = (Handle*)opaqueHandle;
  *sendComm = nullptr;
  if (h->magic == kHandleMagicShm) return shm_connect(dev, opaqueHandle, sendComm);
  if (h->magic != kHandleMagic) { FL_WARN("NET/FuseLink : connect with a handle that listen did not produce"); return ncclInternalError; }
  if (h->stage == 0) {
    Link* lk = new (std::nothrow) Link();
    if (!lk) return ncclSystemError;
    g_live_links.fetch_add(1);
    lk->dev = dev;
    lk->channelId = h->channelId;
    std::lock_guard<std::mutex> g(g_reg_mu);
    auto it = g_listens.find(h->listen_id);
    if (it == g_listens.end()) { delete lk; g_live_links.fetch_sub(1); FL_WARN("NET/FuseLink : connect to a closed listen comm"); return ncclSystemError; }
    it->second->pending.push_back(lk);
    h->stage = 1;
    h->stage_link = lk;
    return ncclSuccess;
  }
  Link* lk = (Link*)h->stage_link;
  int ready;
  {
    std::lock_guard<ShortLock> g(lk->mu);
    ready = lk->send_ready;
  }
  if (ready == 0) return ncclSuccess;  // accept has not happened yet
  if (ready < 0) {                     // the listener went away before it accepted
    h->stage = 0;
    h->stage_link = nullptr;
    link_unref(lk);
    FL_WARN("NET/FuseLink : connect: the listen comm was closed before it accepted");
    return ncclSystemError;
  }
  Comm* c = new (std::nothrow) Comm();
  if (!c) return ncclSystemError;
  c->is_send = 1;
  c->link = lk;
  h->stage = 0;
  h->stage_link = nullptr;
  *sendComm = c;
  return ncclSuccess;
}

ncclResult_t fl_accept(void* listenComm, void** recvComm, ncclNetDeviceHandle_v8_t** /*recvDevComm*/) {
  if (!listenComm || !recvComm) return ncclInvalidArgument;
  ListenComm* lc = (ListenComm*)listenComm;
  *recvComm = nullptr;
  if (lc->magic == kShmListenMagic) return shm_accept((ShmListen*)listenComm, recvComm);
  Link* lk = nullptr;
  {
    std::lock_guard<std::mutex> g(g_reg_mu);
    if (lc->pending.empty()) return ncclSuccess;  // nobody connected yet
    lk = lc->pending.front();
    lc->pending.pop_front();
  }
  Comm* c = new (std::nothrow) Comm();
  if (!c) return ncclSystemError;
  c->is_send = 0;
  c->link = lk;
  {
    std::lock_guard<ShortLock> g(lk->mu);
    lk->send_ready = 1;
  }
  *recvComm = c;
  return ncclSuccess;
}

// Is `fd` a DMA-BUF that holds `size` bytes from `offset` on?  (A dma-buf is a file of the kernel's dmabuf pseudo file
// system: its link in /proc reads "/dmabuf:<name>", and seeking to its end gives its size.)
bool dmabuf_covers(int fd, uint64_t offset, size_t size) {
  char path[64], link[128];
  snprintf(path, sizeof(path), "/proc/self/fd/%d", fd);
  const ssize_t n = readlink(path, link, sizeof(link) - 1);
  if (n <= 0) return false;
  link[n] = 0;
  if (strncmp(link, "/dmabuf:", 8) != 0 && strncmp(link, "anon_inode:dmabuf", 17) != 0) return false;
  const off_t end = lseek(fd, 0, SEEK_END);
  (void)lseek(fd, 0, SEEK_SET);
  return end >= 0 && (uint64_t)end >= offset && (uint64_t)end - offset >= size;
}

ncclResult_t fl_reg_mr_dmabuf(void* comm, void* data, size_t size, int type, uint64_t offset, int fd, void** mhandle) {
  if (!comm || !data || !mhandle || size == 0) return ncclInvalidArgument;
  if (fd >= 0) {
    // A descriptor came with the buffer (plugin.cc:1168, 1278-1280).  It must be what it claims: device memory exported
    // as a DMA-BUF that holds the registered range.  Anything else is refused, not ignored.
    if (type != NCCL_PTR_CUDA || !dmabuf_covers(fd, offset, size)) {
      FL_WARN("NET/FuseLink : regMrDmaBuf: descriptor %d is not a DMA-BUF of device memory that holds %zu bytes from offset %llu", fd, size, (unsigned long long)offset);
      return ncclInvalidArgument;
    }
  }
  Comm* c = (Comm*)comm;
  if (c->magic != kCommMagic) return ncclInvalidArgument;
  const bool wire = c->link->wire != nullptr;   // the other end is another process
  *mhandle = nullptr;
  MemHandle* mh = new (std::nothrow) MemHandle();
  if (!mh) return ncclSystemError;
  mh->type = type;
  if (fd >= 0) {
    mh->dmabuf_fd = dup(fd);   // the caller closes its own
    mh->dmabuf_offset = offset;
    if (mh->dmabuf_fd < 0) { delete mh; return ncclSystemError; }
  }
  if (type == NCCL_PTR_CUDA) {
    // whole allocation around the pointer, as cuMemGetAddressRange in plugin.cc:1194
    void* base = nullptr;
    size_t bsz = 0;
    DeviceScope keep;
    hipPointerAttribute_t attr;
    hipError_t e = hipPointerGetAttributes(&attr, data);
    if (e != hipSuccess) { delete mh; return hip_fail("hipPointerGetAttributes", e); }
    mh->device = g_par.device >= 0 ? g_par.device : attr.device;
    e = hipSetDevice(mh->device);
    if (e != hipSuccess) { delete mh; return hip_fail("hipSetDevice", e); }
    e = hipMemGetAddressRange((hipDeviceptr_t*)&base, &bsz, (hipDeviceptr_t)data);
    if (e != hipSuccess) { delete mh; return hip_fail("hipMemGetAddressRange", e); }
    flh_pool* pool = nullptr;
    ncclResult_t rc = ensure_pool(mh->device, &pool);
    if (rc != ncclSuccess) { delete mh; return rc; }
    // one shared, reference-counted region per base allocation (plugin.cc:1212-1227, 1326)
    int frc = flh_region_acquire(pool, base, bsz, 0, 0, &mh->region);
    if (frc < 0) { delete mh; FL_WARN("NET/FuseLink : region: %s", flh_last_error()); return ncclInternalError; }
    mh->start_addr = (uintptr_t)base;
    mh->size = bsz;
    if (c->is_send || wire) {  // staging (a receiver in another process: its landing windows) is bound at registration time, not on the request path
      std::lock_guard<ShortLock> g(c->link->mu);
      rc = c->is_send ? attach_peer(c->link, mh->device) : wire_recv_setup(c->link, mh->device);
      if (rc != ncclSuccess) { (void)flh_region_release(mh->region); delete mh; return rc; }
      if (wire && !c->is_send) {   // the sender may write into this allocation itself (plugin.cc:1626, 1655: address and rkey go into the descriptor)
        mh->wire_pair = c->link->wire->pair;
        wire_export_mr(mh->wire_pair, base, bsz, &mh->rkey);
      }
    }
  } else if (type == NCCL_PTR_HOST) {
    // page-aligned span, plugin.cc:1181-1182, 1206-1209; host memory is not staged
    const uintptr_t page = 4096;
    const uintptr_t addr = (uintptr_t)data & ~(page - 1);
    const size_t pages = ((uintptr_t)data + size - addr + page - 1) / page;
    mh->start_addr = addr;
    mh->size = pages * page;
  } else {
    delete mh;
    FL_WARN("NET/FuseLink : unsupported pointer type %d", type);
    return ncclInvalidArgument;
  }
  *mhandle = mh;
  return ncclSuccess;
}

ncclResult_t fl_reg_mr_v8(void* comm, void* data, size_t size, int type, void** mhandle) {
  return fl_reg_mr_dmabuf(comm, data, size, type, 0ull, -1, mhandle);  // plugin.cc:1332-1335
}

ncclResult_t fl_dereg_mr(void* /*comm*/, void* mhandle) {
  MemHandle* mh = (MemHandle*)mhandle;
  if (!mh || mh->magic != kMhMagic) return ncclInvalidArgument;
  if (mh->rkey) wire_unexport_mr(mh->wire_pair, mh->rkey);
  if (mh->region) {
    int left = flh_region_release(mh->region);  // destroyed on the last reference, plugin.cc:1347-1403
    if (left < 0) { FL_WARN("NET/FuseLink : region release: %s", flh_last_error()); return ncclInternalError; }
  }
  mh->magic = 0;
  delete mh;
  return ncclSuccess;
}

bool in_handle(const MemHandle* mh, const void* p, size_t n) {
  const uintptr_t a = (uintptr_t)p;
  return a >= mh->start_addr && a + n <= mh->start_addr + mh->size;
}

// Credit row a descriptor asks for: the receiver's row, or one lane named outright.
void wire_credits(const Link* lk, const FifoWire& w, uint32_t* credits) {
  const int lanes = g_par.lanes;
  for (int l = 0; l < FLH_MAX_LANES; ++l) credits[l] = 0;
  if (w.fuselink_offset == -2) {
    for (int l = 0; l < lanes; ++l) credits[l] = w.credits[l];
  } else {
    // the receiver named one lane (fuselink.h:235-237); -1 means the comm's own NIC (plugin.cc:1539-1540)
    const int lane = w.fuselink_offset >= 0 ? w.fuselink_offset % lanes : lk->dev % lanes;
    credits[lane] = 1;
  }
}

void fill_uniform(flh_uniform_params& u, const uint32_t* credits, uint64_t bytes, uint64_t src_base, uint64_t epoch_bytes, uint32_t tile) {
  memset(&u, 0, sizeof(u));
  u.total_bytes = bytes;
  u.src_base = src_base;
  u.epoch_bytes = epoch_bytes;
  u.chunk_bytes = (uint32_t)g_par.chunk;
  u.n_lanes = (uint32_t)g_par.lanes;
  u.tile_bytes = tile;
  for (int l = 0; l < g_par.lanes; ++l) u.credits[l] = credits[l];
}

// copy tile of a launch pair that moves `bytes`: small launches may take a smaller tile, which spreads them over more
// workgroups than there are compute units
uint32_t launch_tile(uint64_t bytes) {
  return g_par.small_tile && bytes < (32ull << 20) ? (uint32_t)g_par.small_tile : FLH_TILE_BYTES;
}

// How the completion of launch `seq` will reach test(): through the completion word (mode 2), through an event that
// the reassembly kernel completes (mode 1), or through an event recorded behind the launch (mode 0, and whatever is
// not a kernel).  Fills the launch's parameters for the first two.
struct Completion {
  hipEvent_t ev = nullptr;   // event to record behind the launch (null: not needed)
  bool rides = false;        // the event was handed to the kernel
};
ncclResult_t launch_event(Peer* pr, uint64_t seq, hipEvent_t* out) {
  const size_t slot = (size_t)((seq - 1) % kEventRing);
  const uint64_t old = pr->ev_seq[slot].load(std::memory_order_acquire);
  if (old && old > pr->done_seq.load(std::memory_order_acquire)) {
    // the ring came round to a launch that nobody has seen complete: wait for it (it is kEventRing launches old)
    FL_HIPCHECK(hipEventSynchronize(pr->evring[slot]));
    uint64_t seen = pr->done_seq.load(std::memory_order_relaxed);
    while (seen < old && !pr->done_seq.compare_exchange_weak(seen, old, std::memory_order_release, std::memory_order_relaxed)) {}
  }
  pr->ev_seq[slot].store(0, std::memory_order_release);
  if (!pr->evring[slot]) FL_HIPCHECK(hipEventCreateWithFlags(&pr->evring[slot], hipEventDisableTiming));
  *out = pr->evring[slot];
  return ncclSuccess;
}
// From this many bytes on a launch is bound by the GPU and not by the host's calls around it.
constexpr uint64_t kEarlyLaunchBytes = 8ull << 20;

void start_stamp(Peer* pr, uint64_t seq, flh_uniform_params& u) {
  if (g_par.completion != 2) return;
  u.d_start_word = pr->d_started;
  u.start_value = (uint32_t)seq;
}
ncclResult_t prepare_completion(Peer* pr, uint64_t seq, uint64_t launch_bytes, flh_uniform_params& last_u, Completion& c) {
  if (g_par.completion == 2) {
    if (launch_bytes < kEarlyLaunchBytes) {
      last_u.d_done_word = pr->d_done;
      last_u.d_done_count = pr->d_count;
      last_u.done_value = (uint32_t)seq;
    }
    return ncclSuccess;
  }
  ncclResult_t rc = launch_event(pr, seq, &c.ev);
  if (rc != ncclSuccess) return rc;
  if (g_par.completion == 1) { last_u.done_event = c.ev; c.rides = true; }
  return ncclSuccess;
}
ncclResult_t finish_completion(Peer* pr, uint64_t seq, const Completion& c) {
  if (!c.ev) return ncclSuccess;
  if (!c.rides) FL_HIPCHECK(hipEventRecord(c.ev, pr->stream));
  pr->ev_seq[(size_t)((seq - 1) % kEventRing)].store(seq, std::memory_order_release);
  pr->last_event_seq.store(seq, std::memory_order_release);
  return ncclSuccess;
}

void note_segment(Peer* pr, uint32_t k, Link* lk, uint32_t first_row, uint32_t n_rows, uint32_t n_req, uint64_t epoch_bytes, const uint64_t* lane_base) {
  LaunchSeg& sg = pr->last.seg[k];
  sg.channelId = lk->channelId;
  sg.first_row = first_row;
  sg.n_rows = n_rows;
  sg.n_req = n_req;
  sg.epoch_bytes = epoch_bytes;
  for (int l = 0; l < FL_NET_MAX_LANES; ++l) sg.lane_base[l] = lane_base ? lane_base[l] : 0;
}

// One matched send on its own (launch_mu held): request -> QP pieces (plugin.cc:1467-1495), each piece -> waves of
// chunks that fit the staging windows, each wave one launch pair.  The last reassembly launch carries the completion.
ncclResult_t launch_transfer(Peer* pr, const Pending& p, uint64_t seq) {
  Link* lk = p.lk;
  uint32_t credits[FLH_MAX_LANES];
  wire_credits(lk, p.w, credits);
  const uint64_t chunk = (uint64_t)g_par.chunk;
  if (pr->wins.cap[0] < chunk) { FL_WARN("NET/FuseLink : staging window smaller than a chunk"); return ncclInternalError; }
  const int nqps = g_par.split_on_qps ? g_par.qps : 1;
  std::vector<int> qoff(nqps), qlen(nqps);
  if (flh_qp_split(p.size, nqps, qoff.data(), qlen.data()) < 0) return ncclInternalError;
  if (p.w.flags & 1u) lk->epoch_bytes = 0;   // the receiver refreshed its lane decision: new credit epoch
  int last_q = -1;
  for (int q = 0; q < nqps; ++q) if (qlen[q] > 0) last_q = q;
  Completion comp;
  for (int q = 0; q < nqps; ++q) {
    uint64_t done = 0;
    const uint64_t piece = (uint64_t)qlen[q];
    while (done < piece) {
      uint64_t wave = (uint64_t)wave_chunks(credits, g_par.lanes, chunk, pr->wins.cap[0], lk->epoch_bytes / chunk) * chunk;
      if (wave > piece - done) wave = piece - done;
      // One credit row, quantum-sized chunks, windows reused from offset 0: the striping launch works out
      // every chunk's lane and window offset itself (and writes the table), the reassembly launch likewise.
      flh_uniform_params u;
      fill_uniform(u, credits, wave, (uint64_t)qoff[q] + done, lk->epoch_bytes, launch_tile(wave));
      start_stamp(pr, seq, u);
      if (g_par.one_pass) {
        // one launch per wave: staged into the windows and written into the receive buffer from the same registers
        if (q == last_q && done + wave == piece) {
          ncclResult_t rc = prepare_completion(pr, seq, wave, u, comp);
          if (rc != ncclSuccess) return rc;
        }
        FL_FLHCHECK(flh_stage_deliver_uniform(p.src, (uint64_t)p.size, p.dst, (uint64_t)p.size, &pr->wins, &u, pr->d_table, pr->d_hdr, pr->d_status, pr->stream));
      } else {
        FL_FLHCHECK(flh_stripe_uniform(p.src, (uint64_t)p.size, &pr->wins, &u, pr->d_table, pr->d_hdr, pr->d_status, pr->stream));
        if (q == last_q && done + wave == piece) {
          ncclResult_t rc = prepare_completion(pr, seq, wave, u, comp);
          if (rc != ncclSuccess) return rc;
        }
        FL_FLHCHECK(flh_reassemble_uniform(p.dst, (uint64_t)p.size, &pr->wins, &u, pr->d_status, pr->stream));
      }
      const uint32_t rows = (uint32_t)((wave + chunk - 1) / chunk);
      pr->last.seq = seq;
      pr->last.engine = false;
      pr->last.n_seg = 1;
      pr->last.n_rows = rows;
      note_segment(pr, 0, lk, 0, rows, 1, lk->epoch_bytes, nullptr);
      lk->last_seq = seq;
      lk->last_engine = false;
      lk->last_first_row = 0;
      lk->last_rows = rows;
      lk->epoch_bytes += wave;
      lk->launches++;
      done += wave;
    }
  }
  return finish_completion(pr, seq, comp);
}

// The same for a receiver in another process (launch_mu held): every wave of chunks is one launch that stages the wave in
// this process's windows and carries it on into a set of the pair's landing windows, a wave of the wire with a launch
// number and a completion of its own.  A wave needs a free landing set; when there is none the send keeps its place (the
// QP piece and the offset it has got to) and *parked says so: the caller queues it again, in front.
ncclResult_t launch_transfer_wire(Peer* pr, Pending& p, WirePair* pair, bool* parked) {
  Link* lk = p.lk;
  *parked = false;
  uint32_t credits[FLH_MAX_LANES];
  wire_credits(lk, p.w, credits);
  const uint64_t chunk = (uint64_t)g_par.chunk;
  if (pr->wins.cap[0] < chunk) { FL_WARN("NET/FuseLink : staging window smaller than a chunk"); return ncclInternalError; }
  const int nqps = g_par.split_on_qps ? g_par.qps : 1;
  std::vector<int> qoff(nqps), qlen(nqps);
  if (flh_qp_split(p.size, nqps, qoff.data(), qlen.data()) < 0) return ncclInternalError;
  if ((p.w.flags & 1u) && p.q_next == 0 && p.q_done == 0) lk->epoch_bytes = 0;   // the receiver refreshed its lane decision: new credit epoch
  int last_q = -1;
  for (int q = 0; q < nqps; ++q) if (qlen[q] > 0) last_q = q;
  for (; p.q_next < nqps; ++p.q_next, p.q_done = 0) {
    const int q = p.q_next;
    const uint64_t piece = (uint64_t)qlen[q];
    while (p.q_done < piece) {
      if (!wire_set_free(pair)) { *parked = true; return ncclSuccess; }
      uint64_t wave = (uint64_t)wave_chunks(credits, g_par.lanes, chunk, pr->wins.cap[0], lk->epoch_bytes / chunk) * chunk;
      if (wave > piece - p.q_done) wave = piece - p.q_done;
      const bool last = q == last_q && p.q_done + wave == piece;
      const uint64_t seq = pr->launch_seq.load(std::memory_order_relaxed) + 1;
      pr->launch_seq.store(seq, std::memory_order_release);
      uint64_t wave_no;
      const uint32_t set = wire_next_set(pair, &wave_no);
      flh_uniform_params u;
      fill_uniform(u, credits, wave, (uint64_t)qoff[q] + p.q_done, lk->epoch_bytes, launch_tile(wave));
      start_stamp(pr, seq, u);
      Completion comp;
      ncclResult_t rc = prepare_completion(pr, seq, wave, u, comp);   // the carrying launch is the last of the path on this side
      if (rc != ncclSuccess) return rc;
      FL_FLHCHECK(flh_stripe_uniform_carry(p.src, (uint64_t)p.size, &pr->wins, &pair->landing_wins[set], &u, pr->d_table, pr->d_hdr, pr->d_status, pr->stream));
      rc = finish_completion(pr, seq, comp);
      if (rc != ncclSuccess) return rc;
      WireFlight f;
      f.engine = false;
      f.seq = seq;
      f.rec.set = set;
      f.rec.n_req = 1;
      f.rec.n_seg = 1;
      f.rec.piece = 1;
      f.rec.offset = (uint64_t)qoff[q] + p.q_done;
      f.rec.last = last ? 1u : 0u;
      f.rec.total_bytes = wave;
      f.rec.req[0] = WaveReq{lk->wire->pair_conn, p.imm, p.fifo_idx, wave};
      f.rec.seg[0] = WaveSeg{lk->epoch_bytes, 1, 0};
      wire_push_flight(pair, f);
      const uint32_t rows = (uint32_t)((wave + chunk - 1) / chunk);
      pr->last.seq = seq;
      pr->last.engine = false;
      pr->last.n_seg = 1;
      pr->last.n_rows = rows;
      note_segment(pr, 0, lk, 0, rows, 1, lk->epoch_bytes, nullptr);
      lk->last_seq = seq;
      lk->last_engine = false;
      lk->last_first_row = 0;
      lk->last_rows = rows;
      lk->epoch_bytes += wave;
      lk->launches++;
      p.q_done += wave;
      p.sreq->seq = seq;
      p.sreq->engine = false;
      p.sreq->wave = wave_no;
    }
  }
  return ncclSuccess;
}

// Does the send have to travel on its own, wave by wave?  Yes if it is split over QPs or if the staging windows
// cannot hold it in one wave from where its connection stands in its credit epoch.
bool needs_waves(const flh_windows& wins, const Pending& p, uint64_t epoch_bytes) {
  if ((g_par.split_on_qps ? g_par.qps : 1) != 1) return true;
  uint32_t credits[FLH_MAX_LANES];
  wire_credits(p.lk, p.w, credits);
  const uint64_t chunk = (uint64_t)g_par.chunk;
  if ((((uint64_t)p.size + chunk - 1) / chunk) > (uint64_t)g_par.max_wave_chunks) return true;
  // where the request's chunks land, from the closed form: it travels in one go if no lane outgrows its window
  FlCreditRow row;
  fl_row_make(credits, (uint32_t)g_par.lanes, row);
  uint64_t lane_bytes[FLH_MAX_LANES];
  uint32_t lane_chunks[FLH_MAX_LANES];
  fl_row_lane_totals(row, epoch_bytes / chunk, (uint64_t)p.size, chunk, lane_bytes, lane_chunks);
  for (int l = 0; l < g_par.lanes; ++l)
    if (lane_bytes[l] > wins.cap[l]) return true;
  return false;
}

// May the send travel in an engine batch?  Small requests only (large ones are bound by the GPU, not by the launch),
// and it must fit one of the engine's window sets in one go.
bool engine_takes(const Peer* pr, const Pending& p, uint64_t epoch_bytes) {
  return pr->engine_ok.load(std::memory_order_acquire) && p.src_dev && p.dst_dev && (int64_t)p.size <= g_par.engine_max_request &&
         !needs_waves(pr->ewins[0], p, epoch_bytes);
}

// The waiting sends work[i ..) that go out as one launch pair (launch_mu held): up to FLH_BATCH_MAX requests in up
// to FLH_SEG_MAX segments.  A segment is a run of requests of one connection under one credit row with no refresh
// inside, every request but its last a whole number of chunks; the segments follow each other in the shared
// windows, and the batch ends where the next request would outgrow a window.  Returns the number of requests taken
// (at least 1: the caller has checked that work[i] alone fits) and fills the batch.
struct BatchBuild {
  flh_batch_params b;
  Link* seg_link[FLH_SEG_MAX];
  uint64_t link_epoch_after[FLH_SEG_MAX];   // the segment's connection's epoch bytes once the segment is scheduled
};
size_t build_batch(Peer* pr, size_t i, BatchBuild& bb, bool engine) {
  const std::vector<Pending>& work = pr->work;
  const flh_windows& wins = engine ? pr->ewins[0] : pr->wins;
  const uint64_t max_chunks = engine ? kEngineRows : (uint64_t)g_par.max_wave_chunks;
  flh_batch_params& b = bb.b;
  memset(&b, 0, sizeof(b));
  const uint64_t chunk = (uint64_t)g_par.chunk;
  b.u.chunk_bytes = (uint32_t)chunk;
  b.u.n_lanes = (uint32_t)g_par.lanes;
  uint64_t closed_end[FLH_MAX_LANES] = {};   // where the closed segments leave every window
  uint64_t seg_bytes = 0;                    // of the open (last) segment
  FlCreditRow row;                           // its credit row
  uint32_t chunks_closed = 0;
  size_t j = i;
  // a batch stays on one wire and travels one way: this process, or one pair of processes, into the posted buffers or through the landing windows
  WirePair* const pair = work[i].lk->wire ? work[i].lk->wire->pair : nullptr;
  const bool direct = work[i].direct;
  while (j < work.size() && b.n_req < (uint32_t)g_par.batch) {
    const Pending& p = work[j];
    if (!(p.src_dev && p.dst_dev) || p.size == 0) break;
    if ((p.lk->wire ? p.lk->wire->pair : nullptr) != pair || p.direct != direct) break;
    // where the request's connection stands in its epoch: behind its earlier segments of this batch, if any
    uint64_t epoch = p.lk->epoch_bytes;
    for (uint32_t k = 0; k < b.n_seg; ++k) if (bb.seg_link[k] == p.lk) epoch = bb.link_epoch_after[k];
    if (p.w.flags & 1u) epoch = 0;
    uint32_t credits[FLH_MAX_LANES];
    wire_credits(p.lk, p.w, credits);
    bool extend = false;
    if (b.n_seg) {
      const uint32_t k = b.n_seg - 1;
      extend = bb.seg_link[k] == p.lk && !(p.w.flags & 1u) && (uint64_t)work[j - 1].size % chunk == 0 &&
               memcmp(b.seg[k].credits, credits, sizeof(credits)) == 0;
    }
    // (whether the request fits is decided below, against what the batch has put into the windows so far; the caller
    // has made sure that work[i] fits empty ones)
    if (engine && (int64_t)p.size > g_par.engine_max_request) break;
    if (!extend && b.n_seg == FLH_SEG_MAX) break;
    // Where would the windows end up?  The open segment grows by the request, or is closed and a new one opens
    // behind it, on every lane at the next multiple of 128 bytes (flh_batch_layout's rule).
    uint64_t base_end[FLH_MAX_LANES], lane_bytes[FLH_MAX_LANES];
    uint32_t lane_chunks[FLH_MAX_LANES];
    FlCreditRow try_row = row;
    uint64_t try_bytes, try_epoch;
    uint32_t chunks_before = chunks_closed;
    if (extend) {
      for (int l = 0; l < FLH_MAX_LANES; ++l) base_end[l] = closed_end[l];
      try_bytes = seg_bytes + (uint64_t)p.size;
      try_epoch = b.seg[b.n_seg - 1].epoch_bytes;
    } else {
      for (int l = 0; l < FLH_MAX_LANES; ++l) base_end[l] = closed_end[l];
      if (b.n_seg) {   // close the open segment
        fl_row_lane_totals(row, b.seg[b.n_seg - 1].epoch_bytes / chunk, seg_bytes, chunk, lane_bytes, lane_chunks);
        for (int l = 0; l < FLH_MAX_LANES; ++l) if (lane_chunks[l]) base_end[l] = (closed_end[l] + 127) / 128 * 128 + lane_bytes[l];
        chunks_before += (uint32_t)((seg_bytes + chunk - 1) / chunk);
      }
      fl_row_make(credits, (uint32_t)g_par.lanes, try_row);
      try_bytes = (uint64_t)p.size;
      try_epoch = epoch;
    }
    fl_row_lane_totals(try_row, try_epoch / chunk, try_bytes, chunk, lane_bytes, lane_chunks);
    bool fits = chunks_before + (try_bytes + chunk - 1) / chunk <= max_chunks;
    for (int l = 0; fits && l < g_par.lanes; ++l)
      if (lane_chunks[l]) fits = (base_end[l] + 127) / 128 * 128 + lane_bytes[l] <= wins.cap[l];
    if (!fits) break;
    uint32_t k;
    if (extend) {
      k = b.n_seg - 1;
      b.seg[k].n_req++;
    } else {
      for (int l = 0; l < FLH_MAX_LANES; ++l) closed_end[l] = base_end[l];
      chunks_closed = chunks_before;
      row = try_row;
      k = b.n_seg++;
      b.seg[k].epoch_bytes = epoch;
      b.seg[k].n_req = 1;
      memcpy(b.seg[k].credits, credits, sizeof(credits));
      bb.seg_link[k] = p.lk;
    }
    seg_bytes = try_bytes;
    bb.link_epoch_after[k] = b.seg[k].epoch_bytes + seg_bytes;
    b.d_src[b.n_req] = p.src;
    b.d_dst[b.n_req] = p.dst;
    b.bytes[b.n_req] = (uint64_t)p.size;
    b.n_req++;
    b.u.total_bytes += (uint64_t)p.size;
    ++j;
  }
  return j - i;
}

// The batch as a launch pair on the peer's stream (engine == false, `seq` its launch number), or handed to the engine
// (engine == true; `seq` then returns the engine's number for the batch).
ncclResult_t launch_batch(Peer* pr, size_t i, size_t n, BatchBuild& bb, bool engine, uint64_t& seq) {
  flh_batch_params& b = bb.b;
  b.u.tile_bytes = launch_tile(b.u.total_bytes);
  uint64_t seg_base[FLH_SEG_MAX][FLH_MAX_LANES];
  if (!engine) FL_FLHCHECK(flh_batch_layout(&b, nullptr, &seg_base[0][0]));
  // a receiver in another process: the batch is a wave of the pair's wire and lands in one of its sets (the caller has
  // made sure that one is free)
  WirePair* const pair = pr->work[i].lk->wire ? pr->work[i].lk->wire->pair : nullptr;
  const bool carry = pair && !pr->work[i].direct;   // (a batch whose posted buffers this process can write itself is staged and delivered here, like a loopback one)
  uint64_t wave_no = 0;
  const uint32_t set = pair ? wire_next_set(pair, &wave_no) : 0;
  if (engine) {
    // batch number k (from 1) takes window set (k - 1) mod sets and slot (k - 1) % kEngineSlots of the tables; the engine
    // lets it in once batch k - sets, the last to use that window set, is complete
    const uint64_t k = pr->engine_submitted.load(std::memory_order_relaxed);
    const uint32_t slot = (uint32_t)(k % kEngineSlots);
    b.u.tile_bytes = FLH_TILE_BYTES;
    uint64_t got = 0;
    const uint64_t starts_before = g_par.trace ? flh_engine_launches(pr->engine) : 0;
    const int64_t t_sub = g_par.trace ? tr_now() : 0;
    const flh_windows* ewin = &pr->ewins[k % (uint64_t)pr->engine_sets];
    const int frc = carry ? flh_engine_submit_wire(pr->engine, FLH_ENGINE_SEND, &b, ewin, &pair->landing_wins[set], pr->d_etable + (size_t)slot * kEngineRows, pr->d_ehdr + slot,
                                                  pr->d_status, &got, &seg_base[0][0])
                         : flh_engine_submit(pr->engine, &b, ewin, pr->d_etable + (size_t)slot * kEngineRows, pr->d_ehdr + slot, pr->d_status, &got, &seg_base[0][0]);
    if (g_par.trace) {   // submits that had to start the resident kernel are counted apart: they pay for a launch
      const int which = flh_engine_launches(pr->engine) != starts_before ? kTrEngineStart : kTrEngineSubmit;
      tr_add(which, 1, tr_now() - t_sub);
    }
    if (frc == FLH_E_NOMEM) return ncclInProgress;   // the descriptor ring is full: the caller takes the launch path for this batch
    if (frc < 0) {
      FL_WARN("NET/FuseLink : engine: %s", flh_last_error());
      pr->engine_ok.store(false, std::memory_order_release);
      return ncclInProgress;
    }
    seq = got;
    pr->engine_reqs_upto[got % kEngineSlots].store(pr->engine_reqs_upto[(got - 1) % kEngineSlots].load(std::memory_order_relaxed) + b.n_req, std::memory_order_relaxed);
    pr->engine_submitted.store(got, std::memory_order_release);
  } else if (carry) {
    start_stamp(pr, seq, b.u);
    Completion comp;
    ncclResult_t rc = prepare_completion(pr, seq, b.u.total_bytes, b.u, comp);   // the carrying launch is the last of the path on this side
    if (rc != ncclSuccess) return rc;
    FL_FLHCHECK(flh_stripe_batch_carry(&b, &pr->wins, &pair->landing_wins[set], pr->d_table, pr->d_hdr, pr->d_status, pr->stream));
    rc = finish_completion(pr, seq, comp);
    if (rc != ncclSuccess) return rc;
  } else if (g_par.one_pass) {
    // one launch stages the batch and writes the receive buffers (this process's, or another's mapped through their
    // registrations)
    start_stamp(pr, seq, b.u);
    Completion comp;
    ncclResult_t rc = prepare_completion(pr, seq, b.u.total_bytes, b.u, comp);
    if (rc != ncclSuccess) return rc;
    FL_FLHCHECK(flh_stage_deliver_batch(&b, &pr->wins, pr->d_table, pr->d_hdr, pr->d_status, pr->stream));
    rc = finish_completion(pr, seq, comp);
    if (rc != ncclSuccess) return rc;
  } else {
    start_stamp(pr, seq, b.u);
    FL_FLHCHECK(flh_stripe_batch(&b, &pr->wins, pr->d_table, pr->d_hdr, pr->d_status, pr->stream));
    Completion comp;
    ncclResult_t rc = prepare_completion(pr, seq, b.u.total_bytes, b.u, comp);
    if (rc != ncclSuccess) return rc;
    FL_FLHCHECK(flh_reassemble_batch(&b, &pr->wins, pr->d_status, pr->stream));
    rc = finish_completion(pr, seq, comp);
    if (rc != ncclSuccess) return rc;
  }
  if (pair) {
    // the wave's record: which receives it answers, each connection's run as one message from its epoch prefix on
    WireFlight f;
    f.engine = engine;
    f.seq = seq;
    f.rec.set = set;
    f.rec.n_req = b.n_req;
    f.rec.n_seg = b.n_seg;
    f.rec.direct = carry ? 0u : 1u;
    f.rec.total_bytes = b.u.total_bytes;
    for (uint32_t q = 0; q < b.n_req; ++q) {
      const Pending& p = pr->work[i + q];
      f.rec.req[q] = WaveReq{p.lk->wire->pair_conn, p.imm, p.fifo_idx, (uint64_t)p.size};
      p.sreq->wave = wave_no;
    }
    for (uint32_t k = 0; k < b.n_seg; ++k) f.rec.seg[k] = WaveSeg{b.seg[k].epoch_bytes, b.seg[k].n_req, 0};
    wire_push_flight(pair, f);
  }
  // bookkeeping: every connection's place in its epoch, what the launch carried
  const uint64_t chunk = (uint64_t)g_par.chunk;
  pr->last.seq = seq;
  pr->last.engine = engine;
  pr->last.n_seg = b.n_seg;
  uint32_t row = 0, q = 0;
  for (uint32_t k = 0; k < b.n_seg; ++k) {
    Link* lk = bb.seg_link[k];
    uint64_t seg_bytes = 0;
    for (uint32_t r = 0; r < b.seg[k].n_req; ++r) seg_bytes += b.bytes[q++];
    const uint32_t rows = (uint32_t)((seg_bytes + chunk - 1) / chunk);
    note_segment(pr, k, lk, row, rows, b.seg[k].n_req, b.seg[k].epoch_bytes, seg_base[k]);
    if (lk->last_seq != seq || lk->last_engine != engine) lk->launches++;
    lk->last_seq = seq;
    lk->last_engine = engine;
    lk->last_first_row = row;
    lk->last_rows = rows;
    lk->epoch_bytes = bb.link_epoch_after[k];
    if (n > 1) lk->batched_requests += b.seg[k].n_req;
    row += rows;
  }
  pr->last.n_rows = row;
  return ncclSuccess;
}

// Launch everything that waits on the peer, in order (launch_mu held).  A failure completes the requests it
// touches with an error, as a queue pair in the error state would (plugin.cc:1839-1861).  Sends to another process
// need a free set of their pair's landing windows; where there is none they, and whatever waits behind them for the
// same pair, go back to the front of the queue.
void flush_pending(Peer* pr) {
  {
    std::lock_guard<ShortLock> g(pr->queue_mu);
    if (pr->pending.empty()) return;
    pr->work.clear();
    pr->work.swap(pr->pending);
    pr->waiting_reqs.store(0, std::memory_order_release);
    pr->waiting_bytes.store(0, std::memory_order_release);
  }
  TraceScope tr(kTrFlush);
  LazyDevice dev(pr->hip_device);
  std::vector<Pending>& work = pr->work;
  if (work.size() > 2) {
    // Sends of several connections arrive interleaved, and every change of connection opens a segment: bring each
    // connection's sends together (in the order the connections first appear, each connection's own order kept), so
    // that a launch holds four connections' requests in four segments instead of closing after eight requests.
    // Requests of different connections are independent of each other, so the order among them is free.
    std::vector<Pending>& sorted = pr->work_sorted;
    sorted.clear();
    sorted.reserve(work.size());
    std::vector<bool>& taken = pr->work_taken;
    taken.assign(work.size(), false);
    for (size_t a = 0; a < work.size(); ++a) {
      if (taken[a]) continue;
      for (size_t b = a; b < work.size(); ++b)
        if (!taken[b] && work[b].lk == work[a].lk) { sorted.push_back(work[b]); taken[b] = true; }
    }
    work.swap(sorted);
  }
  if (g_par.trace) tr_add(kTrRequestsLaunched, (int64_t)work.size(), 0);
  tl_event(3, (uint64_t)work.size());
  std::vector<Pending>& parked = pr->work_sorted;   // (free again) what found no landing set, in order
  parked.clear();
  for (const Pending& q : work) if (q.lk->wire && q.lk->wire->pair) q.lk->wire->pair->blocked = false;
  size_t i = 0;
  while (i < work.size()) {
    ncclResult_t rc = ncclSuccess;
    size_t span = 1;
    Pending& p = work[i];
    WirePair* const pair = p.lk->wire ? p.lk->wire->pair : nullptr;
    if (pair) {
      if (pair->w->failed.load(std::memory_order_acquire) || p.lk->wire->w->recv_closed.load(std::memory_order_acquire)) {
        if (!p.lk->wire->w->recv_closed.load(std::memory_order_acquire)) FL_WARN("NET/FuseLink : a wave to the receiving process was lost: the send fails");
        else FL_WARN("NET/FuseLink : the receiving process closed the connection with a send outstanding");
        p.sreq->fault = 1;
        p.sreq->state.store(kStDoneHost, std::memory_order_release);
        ++i;
        continue;
      }
      if (pair->blocked || !wire_set_free(pair)) {   // no landing set: it keeps its place, and so does what follows it on this wire
        pair->blocked = true;
        parked.push_back(p);
        ++i;
        continue;
      }
    }
    const uint64_t p_epoch = (p.w.flags & 1u) ? 0 : p.lk->epoch_bytes;
    // small requests in device memory go to the engine, batch by batch: no launch, and a number of the engine's own
    bool by_engine = false, wave_by_wave = false;
    uint64_t seq = 0;
    if (rc == ncclSuccess && p.size && g_par.batch >= 2 && p.q_next == 0 && p.q_done == 0 && engine_takes(pr, p, p_epoch)) {
      BatchBuild bb;
      const size_t n = build_batch(pr, i, bb, true);
      if (n) {
        TraceScope trl(kTrLaunch);
        const ncclResult_t erc = launch_batch(pr, i, n, bb, true, seq);
        if (erc == ncclSuccess) { by_engine = true; span = n; }
        else if (erc != ncclInProgress) rc = erc;    // ncclInProgress: the engine could not take it, a launch pair carries it
      }
    }
    if (!by_engine) {
      if (rc == ncclSuccess && !dev.use()) rc = ncclUnhandledCudaError;   // launches need the staging device current
      if (!pair) {   // (waves to another process take their numbers where they are launched: a send may be several)
        seq = pr->launch_seq.load(std::memory_order_relaxed) + 1;   // this launch's number
        pr->launch_seq.store(seq, std::memory_order_release);   // before anything runs: the completion words never run ahead of it
      }
    }
    if (rc == ncclSuccess && !by_engine) {
      if (pair && p.size == 0) {
        // a send of no bytes to another process: a wave with nothing to land, announced in its turn
        uint64_t wave_no;
        WireFlight f;
        f.rec.set = wire_next_set(pair, &wave_no);
        f.rec.n_req = 1;
        f.rec.n_seg = 1;
        f.rec.req[0] = WaveReq{p.lk->wire->pair_conn, p.imm, p.fifo_idx, 0};
        f.rec.seg[0] = WaveSeg{p_epoch, 1, 0};
        wire_push_flight(pair, f);
        p.sreq->wave = wave_no;
        p.sreq->state.store(kStDoneHost, std::memory_order_release);
        ++i;
        continue;
      } else if (!(p.src_dev && p.dst_dev)) {
        // one side is host memory: the copy engine is the wire, nothing is striped
        hipEvent_t ev = nullptr;
        rc = launch_event(pr, seq, &ev);
        hipError_t e = rc == ncclSuccess ? hipMemcpyAsync(p.dst, p.src, (size_t)p.size, hipMemcpyDefault, pr->stream) : hipSuccess;
        if (e != hipSuccess) rc = hip_fail("hipMemcpyAsync", e);
        if (rc == ncclSuccess) { Completion c; c.ev = ev; rc = finish_completion(pr, seq, c); }
      } else if (g_par.batch < 2 || p.q_next || p.q_done || needs_waves(pr->wins, p, p_epoch)) {
        wave_by_wave = true;
      } else {
        BatchBuild bb;
        span = build_batch(pr, i, bb, false);
        TraceScope trl(kTrLaunch);
        // a request on its own takes the single-message kernels: they carry no per-request search and a tenth of the
        // batch kernels' arguments, which is worth a microsecond per kernel on a 64 MiB request
        if (span <= 1) { span = 1; wave_by_wave = true; }
        else {
          if (pair) { seq = pr->launch_seq.load(std::memory_order_relaxed) + 1; pr->launch_seq.store(seq, std::memory_order_release); }
          rc = launch_batch(pr, i, span, bb, false, seq);
        }
      }
      if (wave_by_wave && pair && p.direct) {
        // its posted buffer is mapped here: waves through this process's windows and straight into it, in stream order,
        // then one record for the receiver
        seq = pr->launch_seq.load(std::memory_order_relaxed) + 1;
        pr->launch_seq.store(seq, std::memory_order_release);
        rc = launch_transfer(pr, p, seq);
        if (rc == ncclSuccess) {
          uint64_t wave_no;
          WireFlight f;
          f.seq = seq;
          f.rec.set = wire_next_set(pair, &wave_no);
          f.rec.n_req = 1;
          f.rec.n_seg = 1;
          f.rec.direct = 1;
          f.rec.total_bytes = (uint64_t)p.size;
          f.rec.req[0] = WaveReq{p.lk->wire->pair_conn, p.imm, p.fifo_idx, (uint64_t)p.size};
          f.rec.seg[0] = WaveSeg{p_epoch, 1, 0};
          wire_push_flight(pair, f);
          p.sreq->wave = wave_no;
        }
      } else if (wave_by_wave && pair) {
        bool park = false;
        rc = launch_transfer_wire(pr, p, pair, &park);   // numbers its launches itself, one per wave
        seq = p.sreq->seq;
        if (rc == ncclSuccess && park) {   // part of it is on its way; the rest waits for a landing set, in front
          pair->blocked = true;
          parked.push_back(p);
          ++i;
          continue;
        }
      } else if (wave_by_wave) {
        rc = launch_transfer(pr, p, seq);
      }
    }
    tl_event(4, ((uint64_t)span << 32) | (by_engine ? 0x80000000ull : 0) | (seq & 0x7fffffffull));
    for (size_t k = i; k < i + span; ++k) {
      Pending& q = work[k];
      if (rc == ncclSuccess) {
        q.sreq->seq = seq;
        q.sreq->engine = by_engine;
        q.sreq->state.store(kStLaunched, std::memory_order_release);
        if (q.rreq) {
          q.rreq->seq = seq;
          q.rreq->engine = by_engine;
          q.rreq->state.store(kStLaunched, std::memory_order_release);
        }
      } else {
        q.sreq->fault = 1;
        q.sreq->state.store(kStDoneHost, std::memory_order_release);
        if (q.rreq) {
          q.rreq->fault = 1;
          q.rreq->state.store(kStDoneHost, std::memory_order_release);
        }
        if (pair) pair->w->failed.store(1, std::memory_order_release);   // (its wave, if one was numbered, will never land)
      }
    }
    if (rc != ncclSuccess && !by_engine) {
      // whatever part of the launch was queued is waited for here, so that its number counts as complete and the
      // launches behind it are not held back by one that will never report
      if (dev.use()) (void)hipStreamSynchronize(pr->stream);
      const uint64_t top = pr->launch_seq.load(std::memory_order_relaxed);
      uint64_t seen = pr->done_seq.load(std::memory_order_relaxed);
      while (seen < top && !pr->done_seq.compare_exchange_weak(seen, top, std::memory_order_release, std::memory_order_relaxed)) {}
    }
    i += span;
  }
  work.clear();
  if (!parked.empty()) {
    std::lock_guard<ShortLock> g(pr->queue_mu);
    uint64_t bytes = 0;
    for (const Pending& q : parked) bytes += (uint64_t)q.size;
    pr->pending.insert(pr->pending.begin(), parked.begin(), parked.end());
    pr->waiting_reqs.store(pr->waiting_reqs.load(std::memory_order_relaxed) + (uint32_t)parked.size(), std::memory_order_release);
    pr->waiting_bytes.store(pr->waiting_bytes.load(std::memory_order_relaxed) + bytes, std::memory_order_release);
    parked.clear();
  }
}

ncclResult_t fl_isend(void* sendComm, void* data, int size, int tag, void* mhandle, void** request) {
  if (!sendComm || !request || !mhandle || size < 0 || (size && !data)) return ncclInvalidArgument;
  Comm* c = (Comm*)sendComm;
  MemHandle* mh = (MemHandle*)mhandle;
  if (c->magic != kCommMagic || !c->is_send || mh->magic != kMhMagic) return ncclInvalidArgument;
  Link* lk = c->link;
  WireEnd* const wire = lk->wire;   // non-null: the receiver is another process
  *request = nullptr;
  TraceScope tr(kTrIsend);
  if (wire && mh->type != NCCL_PTR_CUDA) { FL_WARN("NET/FuseLink : the shared-memory wire carries device memory only"); return ncclInvalidUsage; }
  // The connection's lock covers the descriptor match and the bookkeeping only.  The GPU work is queued
  // after it is dropped: one thread drives a send comm (as NCCL's proxy does), so launches on the
  // connection's stream stay in request order, and the receiver's polling never waits behind a launch.
  FifoWire w;
  Request *sreq = nullptr, *rreq = nullptr;
  int rtype = 0;
  uint32_t imm = 0xffffffffu;
  uint64_t fifo_idx = 0;
  ncclResult_t rc = ncclSuccess;
  {
    std::lock_guard<ShortLock> g(lk->mu);
    if (lk->send_ready <= 0) { FL_WARN("NET/FuseLink: isend() called when comm->ready == 0"); return ncclInternalError; }  // plugin.cc:1502
    // wait for the receiver to have posted the matching receive (plugin.cc:1510-1514)
    const int slot = (int)(lk->fifoHead % FL_NET_MAX_REQUESTS);
    FifoSlot& fs = lk->fifo[slot];
    // the descriptor: in this process's ring, or in the shared-memory object the receiving process writes (idx last)
    FifoWire* const fw = wire ? &wire->w->fifo[slot] : &fs.w;
    if (__atomic_load_n(&fw->idx, __ATOMIC_ACQUIRE) != lk->fifoHead + 1) {
      if (wire && wire->w->recv_closed.load(std::memory_order_acquire)) { FL_WARN("NET/FuseLink : the receiving process has closed the connection"); return ncclRemoteError; }
      return ncclSuccess;
    }
    w = *fw;
    if (w.nreqs != 1) { FL_WARN("NET/FuseLink: multi-send not allowed"); return ncclInternalError; }   // plugin.cc:1448-1451
    if (w.tag != (uint32_t)tag) return ncclSuccess;                                                     // plugin.cc:1552
    if (size > w.size) {                                                                                // plugin.cc:1555-1562
      FL_WARN("NET/FuseLink : req tag %x collective mismatch error, local size %d remote size %d", tag, size, w.size);
      return ncclInvalidUsage;
    }
    if (w.size < 0 || w.addr == 0) {                                                                 // plugin.cc:1563-1570
      FL_WARN("NET/FuseLink : posted incorrect receive info: size %d addr %llx", w.size, (unsigned long long)w.addr);
      return ncclInternalError;
    }
    if (size && !in_handle(mh, data, (size_t)size)) { FL_WARN("NET/FuseLink : send buffer outside its registration"); return ncclInvalidArgument; }
    if (wire) {   // the receiver's landing windows, once it has set them up
      bool ready = false;
      rc = wire_send_setup(lk, mh->device, &ready);
      if (rc != ncclSuccess || !ready) return rc;
    }
    sreq = get_request(lk->sreq, lk, kReqSend);
    if (!sreq) return ncclInternalError;                                                                   // plugin.cc:1082-1084
    if (!wire) {
      rreq = fs.rreq;
      rtype = fs.rtype;
    } else {
      rtype = NCCL_PTR_CUDA;
    }
    sreq->size = size;
    if (rreq) rreq->size = size;
    const bool any_dev = mh->type == NCCL_PTR_CUDA || rtype == NCCL_PTR_CUDA;
    if (size && any_dev && !wire) rc = attach_peer(lk, mh->type == NCCL_PTR_CUDA ? mh->device : fs.rdevice);
    if (rc != ncclSuccess) { sreq->type = kReqUnused; return rc; }   // nothing consumed: the descriptor stays posted
    imm = sender_mask(lk);                        // plugin.cc:1441-1447
    if (rreq) rreq->imm = imm;                    // (the immediate data of the write that completes the receive, plugin.cc:1463)
    fifo_idx = lk->fifoHead + 1;
    if (wire) {
      // plugin.cc:1605; the index goes last: once it reads 0 the slot is the receiver's again, and it writes all of it
      memset((void*)fw, 0, offsetof(FifoWire, idx));
      memset((char*)fw + offsetof(FifoWire, idx) + sizeof(uint64_t), 0, sizeof(FifoWire) - offsetof(FifoWire, idx) - sizeof(uint64_t));
      __atomic_store_n(&fw->idx, (uint64_t)0, __ATOMIC_RELEASE);
    } else {
      memset((void*)&fs.w, 0, sizeof(FifoWire));   // plugin.cc:1605
      fs.rreq = nullptr;
    }
    lk->fifoHead++;                              // plugin.cc:1607
    lk->s_inflight++;
  }
  // the receiver's buffer: its address in this process; across processes, where its registration is mapped here (if it
  // is: otherwise null, and the bytes travel through the landing windows)
  uint8_t* dst = wire ? (size ? wire_map_mr(wire->pair, w.rkey, w.addr, (uint64_t)size) : nullptr) : (uint8_t*)(uintptr_t)w.addr;
  const bool src_dev = mh->type == NCCL_PTR_CUDA, dst_dev = rtype == NCCL_PTR_CUDA;
  // the comm's own NIC carried traffic (updateTxChannelActive, fuselink.h:247-252)
  mark_nic_active(lk->dev % g_par.lanes, 1);
  if (!wire && (size == 0 || (!src_dev && !dst_dev))) {
    // host memory is not staged (fuselink.cc:8-13): the wire is a copy
    if (size) memcpy(dst, data, (size_t)size);
    sreq->state.store(kStDoneHost, std::memory_order_release);
    rreq->state.store(kStDoneHost, std::memory_order_release);
  } else {
    // device memory: the launches are made together with the other sends that wait on this GPU
    Peer* pr = lk->peer.load(std::memory_order_acquire);
    Pending p;
    p.lk = lk;
    p.src = (const uint8_t*)data;
    p.dst = dst;
    p.size = size;
    p.src_dev = src_dev;
    p.dst_dev = dst_dev;
    p.w = w;
    p.sreq = sreq;
    p.rreq = rreq;
    p.imm = imm;
    p.fifo_idx = fifo_idx;
    p.direct = wire && dst != nullptr;
    sreq->state.store(kStQueued, std::memory_order_release);
    if (rreq) rreq->state.store(kStQueued, std::memory_order_release);
    tl_event(2, (uint64_t)lk->channelId);
    uint32_t waiting;
    {
      std::lock_guard<ShortLock> g(pr->queue_mu);
      pr->pending.push_back(p);
      waiting = pr->waiting_reqs.load(std::memory_order_relaxed) + 1;
      if (waiting == 1 && g_par.batch_wait_ns) pr->waiting_since.store(tr_now(), std::memory_order_relaxed);
      pr->waiting_reqs.store(waiting, std::memory_order_release);
      pr->waiting_bytes.store(pr->waiting_bytes.load(std::memory_order_relaxed) + (uint64_t)size, std::memory_order_release);
    }
    if ((int)waiting >= g_par.batch) {   // a full launch waits (NCCL_FUSELINK_BATCH=1: every send is launched here)
      if (g_par.batch < 2) {
        std::lock_guard<std::mutex> g(pr->launch_mu);
        flush_pending(pr);
      } else if (!pr->launching.load(std::memory_order_relaxed) && pr->launch_mu.try_lock()) {   // if another thread is launching, the next poll takes care of it
        pr->launching.store(true, std::memory_order_relaxed);
        flush_pending(pr);
        pr->launching.store(false, std::memory_order_relaxed);
        pr->launch_mu.unlock();
      }
    }
  }
  *request = sreq;
  return ncclSuccess;
}

ncclResult_t fl_irecv(void* recvComm, int n, void** data, int* sizes, int* tags, void** mhandles, void** request) {
  if (!recvComm || !request || !data || !sizes || !tags || !mhandles) return ncclInvalidArgument;
  Comm* c = (Comm*)recvComm;
  if (c->magic != kCommMagic || c->is_send) return ncclInvalidArgument;
  *request = nullptr;
  if (n > FL_NET_MAX_RECVS) return ncclInternalError;                       // plugin.cc:1683
  if (n != 1) { FL_WARN("NET/FuseLink: multi recv not allowed"); return ncclInternalError; }  // plugin.cc:1873-1880
  MemHandle* mh = (MemHandle*)mhandles[0];
  if (!mh || mh->magic != kMhMagic || sizes[0] < 0 || !data[0]) return ncclInvalidArgument;
  if (sizes[0] && !in_handle(mh, data[0], (size_t)sizes[0])) { FL_WARN("NET/FuseLink : receive buffer outside its registration"); return ncclInvalidArgument; }
  Link* lk = c->link;
  WireEnd* const wire = lk->wire;   // non-null: the sender is another process
  if (wire && mh->type != NCCL_PTR_CUDA) { FL_WARN("NET/FuseLink : the shared-memory wire carries device memory only"); return ncclInvalidUsage; }
  TraceScope tr(kTrIrecv);
  if (wire && wire->pair) (void)wire_progress_recv(wire->pair);   // landing sets whose waves have been delivered go back
  std::lock_guard<ShortLock> g(lk->mu);
  if (wire) {
    ncclResult_t rc = wire_recv_setup(lk, mh->device);
    if (rc != ncclSuccess) return rc;
  }
  const int slot = (int)(lk->fifoTail % FL_NET_MAX_REQUESTS);
  FifoSlot& fs = lk->fifo[slot];
  bool refreshed = false;
  if (lk->r_finished % g_par.refresh_batch == 0 || !lk->have_decision) {   // plugin.cc:1700
    // only when everything received so far has been consumed (plugin.cc:1704-1709)
    if (lk->r_inflight != 0) return ncclSuccess;
    if (g_par.policy == 0) {
      lk->fuselink_offset = lk->channelId % g_par.lanes;                     // refreshRxComm, fuselink.h:235-237
    } else {
      lk->fuselink_offset = -2;
      current_credits(lk->dev % g_par.lanes, lk->tx_available, wire == nullptr, lk->credits);   // plugin.cc:1710
    }
    lk->have_decision = true;
    lk->refreshes++;
    refreshed = true;
  }
  Request* rreq = get_request(lk->rreq, lk, kReqRecv);
  if (!rreq) return ncclInternalError;                                         // plugin.cc:1082-1084
  // descriptor ring full: in this process the head says so; across processes the sender clears a slot when it matches
  // it (plugin.cc:1605), and this side's note of the slot goes when its wave has been delivered
  if (wire ? (fs.rreq || __atomic_load_n(&wire->w->fifo[slot].idx, __ATOMIC_ACQUIRE) != 0) : lk->fifoTail - lk->fifoHead >= FL_NET_MAX_REQUESTS) {
    rreq->type = kReqUnused;
    return ncclSuccess;
  }
  rreq->state.store(kStPosted, std::memory_order_relaxed);
  // ncclIbPostFifo, plugin.cc:1616-1677
  fs.w.addr = (uint64_t)(uintptr_t)data[0];
  fs.w.size = sizes[0];
  fs.w.rkey = !wire ? 1u : (mh->wire_pair == wire->pair ? mh->rkey : 0u);   // across processes: the key to write the buffer directly, if there is one
  fs.w.nreqs = (uint32_t)n;
  fs.w.tag = (uint32_t)tags[0];
  fs.w.fuselink_offset = lk->fuselink_offset;
  memcpy(fs.w.credits, lk->credits, sizeof(fs.w.credits));
  fs.w.flags = refreshed ? 1u : 0u;
  fs.rreq = rreq;
  fs.rtype = mh->type;
  fs.rdevice = mh->device;
  tl_event(1, (uint64_t)lk->channelId);
  if (wire) {
    // this side keeps its note of the slot (the receive it belongs to, the credit row it asked for); the descriptor
    // itself goes into the sender's view, its index last
    FifoWire& out = wire->w->fifo[slot];
    fs.w.idx = 0;
    out = fs.w;
    fs.w.idx = lk->fifoTail + 1;
    __atomic_store_n(&out.idx, lk->fifoTail + 1, __ATOMIC_RELEASE);   // what the sender waits for (plugin.cc:1632)
  } else {
    fs.w.idx = lk->fifoTail + 1;   // written last: it is what the sender waits for (plugin.cc:1632)
  }
  lk->fifoTail++;
  lk->r_inflight++;
  *request = rreq;
  return ncclSuccess;
}

ncclResult_t fl_iflush(void* recvComm, int /*n*/, void** /*data*/, int* /*sizes*/, void** /*mhandles*/, void** request) {
  // A receive completes only after its reassembly kernel has finished on the GPU that owns the
  // buffer, so there is nothing left to flush; the reference too returns without a request when
  // its flush is disabled, the default (plugin.cc:887, 1772).
  if (!recvComm || !request) return ncclInvalidArgument;
  *request = nullptr;
  return ncclSuccess;
}

// Is launch `seq` of the peer complete?  Launches run in order on one stream, so a launch is complete once a later
// one is.  Mode 2 reads the completion word: a plain load of pinned memory.  Launches whose completion is an event
// (the other modes, and whatever is not a kernel) are asked through the runtime.
// Highest launch number that the completion words say is complete: the launch whose reassembly kernel reported itself
// finished, or the one before the launch whose striping kernel has started, whichever is later.  The acquire loads
// pair with the kernels' release stores at system scope.
uint64_t words_complete(Peer* pr) {
  const uint32_t done = __atomic_load_n(pr->h_done, __ATOMIC_ACQUIRE);
  const uint32_t started = __atomic_load_n(pr->h_started, __ATOMIC_ACQUIRE);
  const uint64_t top = pr->launch_seq.load(std::memory_order_acquire);
  auto lift = [top](uint32_t word) {   // the word holds the low half of a launch number at or below `top`
    if (word == 0) return (uint64_t)0;
    uint64_t v = (top & ~0xffffffffull) | word;
    if (v > top) v = v >= (1ull << 32) ? v - (1ull << 32) : 0;
    return v;
  };
  const uint64_t a = lift(done), b = lift(started);
  return a > (b ? b - 1 : 0) ? a : (b ? b - 1 : 0);
}

// Is launch `seq` of the peer complete?  Launches run in order on one stream, so a launch is complete once a later
// one is.  Mode 2 reads the completion words: plain loads of pinned memory.  Launches whose completion is an event
// (the other modes, whatever is not a kernel, a large launch that nothing followed) are asked through the runtime.
ncclResult_t launch_complete(Peer* pr, uint64_t seq, bool* done) {
  *done = false;
  uint64_t seen = pr->done_seq.load(std::memory_order_acquire);
  if (seq <= seen) { *done = true; return ncclSuccess; }
  if (g_par.completion == 2) {
    const uint64_t upto = words_complete(pr);
    if (upto > seen) {
      while (seen < upto && !pr->done_seq.compare_exchange_weak(seen, upto, std::memory_order_release, std::memory_order_relaxed)) {}
      if (seq <= upto) { *done = true; return ncclSuccess; }
    }
  }
  const size_t slot = (size_t)((seq - 1) % kEventRing);
  if (pr->ev_seq[slot].load(std::memory_order_acquire) != seq) {
    // No event stands for this launch.  If it is a large launch of mode 2 and the newest on the stream, nothing will
    // report it: put an event behind it now (the queue ends there, so the event's packet delays no kernel).
    if (g_par.completion != 2 || seq != pr->launch_seq.load(std::memory_order_acquire) || !pr->launch_mu.try_lock()) return ncclSuccess;
    ncclResult_t rc = ncclSuccess;
    if (seq == pr->launch_seq.load(std::memory_order_relaxed) && pr->ev_seq[slot].load(std::memory_order_relaxed) != seq &&
        words_complete(pr) < seq) {
      DeviceScope keep;
      hipEvent_t ev = nullptr;
      hipError_t e = hipSetDevice(pr->hip_device);
      if (e != hipSuccess) rc = hip_fail("hipSetDevice", e);
      if (rc == ncclSuccess) rc = launch_event(pr, seq, &ev);
      if (rc == ncclSuccess) { Completion c; c.ev = ev; rc = finish_completion(pr, seq, c); }
    }
    pr->launch_mu.unlock();
    return rc;   // the next poll asks the event (or finds the words)
  }
  hipError_t e = hipEventQuery(pr->evring[slot]);
  if (e == hipErrorNotReady) return ncclSuccess;
  if (e != hipSuccess) return hip_fail("hipEventQuery", e);
  seen = pr->done_seq.load(std::memory_order_relaxed);
  while (seen < seq && !pr->done_seq.compare_exchange_weak(seen, seq, std::memory_order_release, std::memory_order_relaxed)) {}
  *done = true;
  return ncclSuccess;
}

// Engine batches handed over and not yet reported complete.
uint64_t engine_in_flight(Peer* pr) {
  if (!pr->engine || !pr->engine_ok.load(std::memory_order_acquire)) return 0;   // an engine that went down holds nothing back
  const uint64_t sub = pr->engine_submitted.load(std::memory_order_acquire), done = flh_engine_completed(pr->engine);
  return sub > done ? sub - done : 0;
}

// Requests in the engine batches that are not yet reported complete.
uint64_t engine_requests_in_flight(Peer* pr) {
  if (!pr->engine || !pr->engine_ok.load(std::memory_order_acquire)) return 0;
  const uint64_t sub = pr->engine_submitted.load(std::memory_order_acquire), done = flh_engine_completed(pr->engine);
  if (sub <= done || sub - done >= kEngineSlots) return 0;
  return pr->engine_reqs_upto[sub % kEngineSlots].load(std::memory_order_relaxed) - pr->engine_reqs_upto[done % kEngineSlots].load(std::memory_order_relaxed);
}

// Launches of the peer that have been queued and are not known to be complete.
uint64_t launches_in_queue(Peer* pr) {
  uint64_t done = pr->done_seq.load(std::memory_order_acquire);
  const uint64_t top = pr->launch_seq.load(std::memory_order_acquire);
  if (g_par.completion == 2) {
    const uint64_t upto = words_complete(pr);
    if (upto > done) done = upto;
  }
  return top > done ? top - done : 0;
}

// Is the wave's GPU work through?  (*rc: the engine that held it went down, or the runtime failed.)
bool wire_flight_complete(Peer* pr, const WireFlight& f, ncclResult_t* rc) {
  *rc = ncclSuccess;
  if (f.seq == 0) return true;
  if (f.engine) {
    if (flh_engine_completed(pr->engine) >= f.seq) return true;
    if (flh_engine_error(pr->engine) == 0) return false;
    *rc = ncclRemoteError;
    return true;
  }
  bool complete = false;
  *rc = launch_complete(pr, f.seq, &complete);
  return complete || *rc != ncclSuccess;
}

// One announced wave (rx_mu and the staging side's launch_mu held): the receives it answers, the same batch the sender
// built -- each connection's run as one message from its epoch prefix on, under the credit row this side put into the
// descriptors -- handed to this process's engine or launched, out of the landing set the wave lies in.
ncclResult_t wire_deliver(WirePair* p, const ShmWave& wv, WireFlight& f) {
  Peer* pr = p->peer;
  const uint32_t n_req = wv.n_req, n_seg = wv.n_seg;
  if (n_req < 1 || n_req > FLH_BATCH_MAX || n_seg < 1 || n_seg > FLH_SEG_MAX || wv.set >= (uint32_t)p->sets || (wv.piece && n_req != 1)) {
    FL_WARN("NET/FuseLink : a wave record that makes no sense (%u requests, %u segments, set %u)", n_req, n_seg, wv.set);
    return ncclInternalError;
  }
  flh_batch_params b;
  memset(&b, 0, sizeof(b));
  b.u.chunk_bytes = (uint32_t)g_par.chunk;
  b.u.n_lanes = (uint32_t)g_par.lanes;
  b.u.tile_bytes = FLH_TILE_BYTES;
  b.n_req = n_req;
  b.n_seg = n_seg;
  Request* reqs[FLH_BATCH_MAX];
  Link* links[FLH_BATCH_MAX];
  uint32_t q = 0;
  uint64_t sum = 0;
  bool small = true;
  for (uint32_t k = 0; k < n_seg; ++k) {
    const uint32_t nq = wv.seg[k].n_req;
    if (nq == 0 || q + nq > n_req) { FL_WARN("NET/FuseLink : a wave whose segments do not add up to its requests"); return ncclInternalError; }
    b.seg[k].epoch_bytes = wv.seg[k].epoch_bytes;
    b.seg[k].n_req = nq;
    for (uint32_t i = 0; i < nq; ++i, ++q) {
      const WaveReq& wr = wv.req[q];
      Link* lk = wr.conn < kPairConns ? p->conns[wr.conn].load(std::memory_order_acquire) : nullptr;
      if (!lk) { FL_WARN("NET/FuseLink : a wave for connection %u, which this process does not have", wr.conn); return ncclInternalError; }
      std::lock_guard<ShortLock> g(lk->mu);
      FifoSlot& fs = lk->fifo[(wr.fifo_idx - 1) % FL_NET_MAX_REQUESTS];
      if (!fs.rreq || fs.w.idx != wr.fifo_idx) { FL_WARN("NET/FuseLink : a wave of request %llu arrived, which no posted receive is waiting for", (unsigned long long)wr.fifo_idx); return ncclInternalError; }
      const uint64_t at = wv.piece ? wv.offset : 0;
      if (at + wr.bytes > (uint64_t)fs.w.size) { FL_WARN("NET/FuseLink : a wave past the end of the posted buffer"); return ncclInvalidUsage; }
      uint32_t credits[FLH_MAX_LANES];
      wire_credits(lk, fs.w, credits);
      if (i == 0) memcpy(b.seg[k].credits, credits, sizeof(credits));
      else if (links[q - 1] != lk || memcmp(b.seg[k].credits, credits, sizeof(credits)) != 0) {
        FL_WARN("NET/FuseLink : request %u of a wave does not belong to its segment's connection and credit row", q);
        return ncclInvalidUsage;
      }
      reqs[q] = fs.rreq;
      links[q] = lk;
      b.d_dst[q] = (void*)(uintptr_t)fs.w.addr;
      b.bytes[q] = wr.bytes;
      sum += wr.bytes;
      if ((int64_t)wr.bytes > g_par.engine_max_request) small = false;
      fs.rreq->size += (int)wr.bytes;
      fs.rreq->imm = wr.imm;
      if (!wv.piece || wv.last) { fs.rreq = nullptr; fs.w.idx = 0; }   // the slot's note goes: it may be posted again
    }
  }
  if (q != n_req || sum != wv.total_bytes) { FL_WARN("NET/FuseLink : a wave's requests do not add up to its bytes"); return ncclInvalidUsage; }
  b.u.total_bytes = sum;
  const flh_windows* landing = &p->landing_wins[wv.set];
  const uint64_t chunk = (uint64_t)g_par.chunk;
  bool by_engine = false;
  uint64_t seq = 0;
  ncclResult_t rc = ncclSuccess;
  const bool nothing = sum == 0 || wv.direct != 0;
  if (nothing) {
    // a send of no bytes, or bytes that the sender has written into the posted buffers itself (they were in memory
    // before it announced the wave): nothing to deliver
  } else {
    uint64_t rows = 0;
    for (uint32_t i = 0; i < n_req; ++i) rows += (b.bytes[i] + chunk - 1) / chunk;
    if (!wv.piece && small && rows <= kEngineRows && pr->engine_ok.load(std::memory_order_acquire)) {
      uint64_t got = 0;
      const int frc = flh_engine_submit_wire(pr->engine, FLH_ENGINE_RECV, &b, landing, nullptr, nullptr, nullptr, pr->d_status, &got, nullptr);
      if (frc == FLH_OK) {
        by_engine = true;
        seq = got;
        pr->engine_reqs_upto[got % kEngineSlots].store(pr->engine_reqs_upto[(got - 1) % kEngineSlots].load(std::memory_order_relaxed) + n_req, std::memory_order_relaxed);
        pr->engine_submitted.store(got, std::memory_order_release);
      } else if (frc != FLH_E_NOMEM) {
        FL_WARN("NET/FuseLink : engine: %s", flh_last_error());
        pr->engine_ok.store(false, std::memory_order_release);
      }
    }
    if (!by_engine) {
      DeviceScope keep;
      hipError_t he = hipSetDevice(pr->hip_device);
      if (he != hipSuccess) rc = hip_fail("hipSetDevice", he);
      seq = pr->launch_seq.load(std::memory_order_relaxed) + 1;
      pr->launch_seq.store(seq, std::memory_order_release);
      Completion comp;
      if (rc == ncclSuccess) {
        if (n_req == 1) {
          // one request (or a piece of one): the single-message kernel, under the credit row of its descriptor
          flh_uniform_params u;
          fill_uniform(u, b.seg[0].credits, sum, wv.piece ? wv.offset : 0, b.seg[0].epoch_bytes, launch_tile(sum));
          start_stamp(pr, seq, u);
          rc = prepare_completion(pr, seq, sum, u, comp);
          const uint64_t posted = (uint64_t)(wv.piece ? wv.offset : 0) + sum;   // (checked against the posted size above)
          if (rc == ncclSuccess && flh_reassemble_uniform(b.d_dst[0], posted, landing, &u, pr->d_status, pr->stream) < 0) { FL_WARN("NET/FuseLink : %s", flh_last_error()); rc = ncclUnhandledCudaError; }
        } else {
          b.u.tile_bytes = launch_tile(sum);
          start_stamp(pr, seq, b.u);
          rc = prepare_completion(pr, seq, sum, b.u, comp);
          if (rc == ncclSuccess && flh_reassemble_batch(&b, landing, pr->d_status, pr->stream) < 0) { FL_WARN("NET/FuseLink : %s", flh_last_error()); rc = ncclUnhandledCudaError; }
        }
      }
      if (rc == ncclSuccess) rc = finish_completion(pr, seq, comp);
      if (rc != ncclSuccess) {
        // whatever was queued is waited for, so that the number counts as complete and holds nothing back
        (void)hipStreamSynchronize(pr->stream);
        uint64_t seen = pr->done_seq.load(std::memory_order_relaxed);
        while (seen < seq && !pr->done_seq.compare_exchange_weak(seen, seq, std::memory_order_release, std::memory_order_relaxed)) {}
      }
    }
  }
  f.engine = by_engine;
  f.seq = nothing || rc != ncclSuccess ? 0 : seq;
  if (wv.piece && !wv.last && rc == ncclSuccess) return ncclSuccess;   // the request's later pieces complete it
  for (uint32_t i = 0; i < n_req; ++i) {
    Request* r = reqs[i];
    r->seq = seq;
    r->engine = by_engine;
    if (rc != ncclSuccess) r->fault = 1;
    r->state.store(nothing || rc != ncclSuccess ? kStDoneHost : kStLaunched, std::memory_order_release);
  }
  return rc;
}

ncclResult_t fl_test(void* request, int* done, int* sizes) {
  if (!request || !done) return ncclInvalidArgument;
  Request* r = (Request*)request;
  if (r->magic != kReqMagic || r->type == kReqUnused) { FL_WARN("NET/FuseLink : test on a request that is not in flight"); return ncclInternalError; }
  *done = 0;
  Link* lk = r->link;
  TraceScope tr(kTrTest);
  WirePair* const pair = lk->wire ? lk->wire->pair : nullptr;   // non-null: the other end is another process
  // The other end is another process: whoever polls a receive takes the waves that have been announced off the wire,
  // whoever polls a send announces the waves that have landed -- also while its own request still waits for a landing
  // set, which only comes back once the receiver has seen the waves before it.
  if (pair && r->type == kReqRecv) (void)wire_progress_recv(pair);
  if (pair && r->type == kReqSend) (void)wire_publish(pair);
  // the request is polled without the connection's lock: only the thread that drives this comm tests its requests
  int st = r->state.load(std::memory_order_acquire);
  if (st == kStPosted || st == 0) {   // a receive whose send has not been matched yet
    if (!lk->wire) return ncclSuccess;
    // the sender is another process: has a wave been lost on the way, or has the sender gone?
    const bool lost = pair && pair->w->failed.load(std::memory_order_acquire);
    if (!lost) {
      if (!lk->wire->w->send_closed.load(std::memory_order_acquire)) return ncclSuccess;
      // (what it announced before it left is still delivered: look once more before giving up)
      if (pair) (void)wire_progress_recv(pair);
      st = r->state.load(std::memory_order_acquire);
      if ((st == kStPosted || st == 0) && pair) {
        const uint64_t taken = pair->rx_taken.load(std::memory_order_acquire);
        if (pair->w->wave[taken % kPairWaves].seq.load(std::memory_order_acquire) == taken + 1) return ncclSuccess;   // an announced wave has yet to be taken off the wire
      }
    }
    if (st == kStPosted || st == 0) {
      FL_WARN("NET/FuseLink : %s", lost ? "a wave from the sending process was lost" : "the sending process closed the connection with a receive outstanding");
      r->fault = 1;
      st = kStDoneHost;
    }
  }
  Peer* pr = lk->peer.load(std::memory_order_acquire);
  // Matched sends wait so that those that arrive together -- on this connection and on the others that stage on
  // the same GPU -- can share a launch.  They go out when a test finds the GPU short of work: fewer than two
  // launches in its queue and something waiting, whichever request is being polled.  While two launches or more are
  // queued the GPU is not waiting for the host, and holding the sends back costs them nothing but lets the next
  // launch carry more of them; a full launch's worth (NCCL_FUSELINK_BATCH) never waits (isend launches it).
  if (pr && pr->waiting_reqs.load(std::memory_order_acquire) != 0) {
    // a launch whose completion comes from an event is only known complete once its own requests are polled: it
    // must not hold anything back
    const bool events_out = pr->last_event_seq.load(std::memory_order_acquire) > pr->done_seq.load(std::memory_order_acquire);
    const uint64_t in_flight = launches_in_queue(pr) + engine_in_flight(pr);
    bool go = events_out || g_par.completion != 2 || in_flight < (uint64_t)g_par.queue_depth ||
              (in_flight < (uint64_t)pr->engine_sets &&
               ((g_par.eager_batch > 0 && pr->waiting_reqs.load(std::memory_order_acquire) >= (uint32_t)g_par.eager_batch) ||
                engine_requests_in_flight(pr) < (uint64_t)g_par.light_load));
    // small sends wait a moment for company: a launch pair costs the host as much as ten requests do
    if (go && g_par.batch_wait_ns && pr->waiting_bytes.load(std::memory_order_acquire) < kEarlyLaunchBytes &&
        pr->waiting_reqs.load(std::memory_order_acquire) < (uint32_t)g_par.batch &&
        tr_now() - pr->waiting_since.load(std::memory_order_relaxed) < g_par.batch_wait_ns)
      go = false;
    if (go && !pr->launching.load(std::memory_order_relaxed)) {
      if (pr->launch_mu.try_lock()) {   // if another thread is launching, it or the next poll takes care of it
        pr->launching.store(true, std::memory_order_relaxed);
        flush_pending(pr);
        pr->launching.store(false, std::memory_order_relaxed);
        pr->launch_mu.unlock();
      }
      st = r->state.load(std::memory_order_acquire);
    }
  }
  if (st == kStQueued) return ncclSuccess;
  // Timing experiment, behind the test-hook switch: report a send complete as soon as its batch has been handed over.
  // Unsafe for a real caller (the source may still be read), but it bounds from above what any earlier completion of
  // sends -- when their bytes are staged, say -- could be worth to the request rate.
  if (g_par.test_early_send && st == kStLaunched && r->type == kReqSend && !pair) st = kStDoneHost;
  if (st == kStLaunched && r->engine) {
    // the engine stores the number of the last complete batch to a pinned word: a plain load, as for the launches' words
    const uint64_t e_done = flh_engine_completed(pr->engine);
    if (g_par.trace >= 2) {
      uint64_t seen = pr->tl_engine_seen.load(std::memory_order_relaxed);
      while (e_done > seen && !pr->tl_engine_seen.compare_exchange_weak(seen, e_done, std::memory_order_relaxed)) {}
      if (e_done > seen) tl_event(6, e_done);
    }
    if (e_done < r->seq) {
      if (flh_engine_error(pr->engine) == 0) {
        // an engine whose time as a resident ran out leaves between two batches; with nothing further to submit, the
        // thread that waits for one of them starts the next engine (two loads of host memory to find out)
        if (flh_engine_needs_start(pr->engine) && pr->launch_mu.try_lock()) {
          LazyDevice dev(pr->hip_device);
          if (dev.use() && flh_engine_poke(pr->engine) < 0) FL_WARN("NET/FuseLink : engine: %s", flh_last_error());
          pr->launch_mu.unlock();
        }
        return ncclSuccess;
      }
      // the engine went down on a wait that ran out: what it still held is lost, later traffic travels by launches
      pr->engine_ok.store(false, std::memory_order_release);
      FL_WARN("NET/FuseLink : the lane engine stopped with an error; channel %d falls back to launches", lk->channelId);
      r->fault = 1;
    }
  } else if (st == kStLaunched) {
    bool complete = false;
    ncclResult_t rc = launch_complete(pr, r->seq, &complete);
    if (rc != ncclSuccess || !complete) return rc;
  }
  if (pair && r->type == kReqSend && !r->fault) {
    // A send to another process is reported once its wave has been announced there (like an RDMA write, complete when
    // the bytes are in the receiver's memory, plugin.cc:1453-1465): announce what has landed, in order.
    ncclResult_t prc = wire_publish(pair);
    if (prc != ncclSuccess || pair->w->failed.load(std::memory_order_acquire)) {
      FL_WARN("NET/FuseLink : a wave to the receiving process was lost");
      r->fault = 1;
    } else if (pair->tx_published.load(std::memory_order_acquire) < r->wave) {
      if (!lk->wire->w->recv_closed.load(std::memory_order_acquire)) return ncclSuccess;   // waves before it are still landing
      FL_WARN("NET/FuseLink : the receiving process closed the connection with a wave outstanding");
      r->fault = 1;
    }
  }
  if (g_par.trace) tr_add(kTrTestDone, 1, 0);
  tl_event(5, ((uint64_t)r->seq << 16) | (r->engine ? 0x8000u : 0u) | ((uint64_t)(lk->channelId & 0x3fff) << 1) | (r->type == kReqRecv ? 1u : 0u));
  ncclResult_t result = ncclSuccess;
  {
    std::lock_guard<ShortLock> g(lk->mu);
    if (r->fault) {
      // Failed completion (plugin.cc:1839-1861).  The reference returns here with the request still allocated and its
      // counters untouched: its communicator is dead from then on.  Here the connection lives on (an engine that went
      // down hands its traffic to launches), so the request is freed and counted like any other: a request that stayed
      // in flight would hold every later refresh back (r_inflight != 0 on a batch boundary) and leak its slot.
      FL_WARN("NET/FuseLink : Got completion with error, channel %d, %s", lk->channelId, r->type == kReqSend ? "Send" : "Recv");
      result = ncclRemoteError;
    } else if (st == kStLaunched && pr && __atomic_load_n(pr->h_status, __ATOMIC_ACQUIRE) != 0) {
      // A kernel refused a chunk that would have left its window or buffer (the host sizes every launch so that this
      // cannot happen; the check is the safety net).  The first request completed after the refusal reports it, once,
      // and is freed like any other; the word is cleared so that later traffic is not condemned with it.
      const int32_t code = __atomic_exchange_n(pr->h_status, 0, __ATOMIC_ACQ_REL);
      if (code != 0) {
        FL_WARN("NET/FuseLink : a chunk fell outside its staging window or buffer (status %d)", code);
        result = ncclInternalError;
      }
    }
    *done = result == ncclSuccess ? 1 : 0;                    // plugin.cc:1807-1823
    if (r->type == kReqSend) { lk->s_finished++; lk->s_inflight--; }
    if (r->type == kReqRecv) {
      mark_nic_active(lk->dev % g_par.lanes, 0);   // updateRxChannelActive, fuselink.h:254-259
      if (result == ncclSuccess) lk->tx_available = r->imm;   // comm->txAvailable = wc->imm_data, plugin.cc:1884-1885
      lk->r_finished++;
      lk->r_inflight--;
      if (sizes) sizes[0] = r->size;   // the reference leaves 0 here (plugin.cc:1726, 1882)
    }
    r->type = kReqUnused;                                     // ncclIbFreeRequest, plugin.cc:1086-1090
  }
  // a receive that is through frees its wave's landing set at the next look; look now, the sender may be waiting for it
  if (pair && !lk->wire->is_send) (void)wire_progress_recv(pair);
  return result;
}

ncclResult_t close_comm(void* comm, int want_send) {
  Comm* c = (Comm*)comm;
  if (!c) return ncclSuccess;
  if (c->magic != kCommMagic || c->is_send != want_send) return ncclInvalidArgument;
  Link* lk = c->link;
  if (lk->wire && lk->wire->pair) {
    // what this end still owes the other process goes out before the end is marked closed: a sender announces the
    // waves that have landed, a receiver hands back the landing sets of the waves it has delivered
    WirePair* pair = lk->wire->pair;
    const int64_t until = tr_now() + 2000000000ll;
    if (want_send) {
      for (;;) {
        (void)wire_publish(pair);
        bool empty;
        { std::lock_guard<std::mutex> g(pair->tx_mu); empty = pair->tx_flights.empty(); }
        if (empty || pair->w->failed.load(std::memory_order_acquire) || tr_now() > until) break;
      }
    } else {
      (void)wire_progress_recv(pair);
    }
  }
  c->magic = 0;
  delete c;
  link_unref(lk);
  return ncclSuccess;
}
ncclResult_t fl_close_send(void* sendComm) { return close_comm(sendComm, 1); }
ncclResult_t fl_close_recv(void* recvComm) { return close_comm(recvComm, 0); }

ncclResult_t fl_close_listen(void* listenComm) {
  ListenComm* lc = (ListenComm*)listenComm;
  if (!lc) return ncclSuccess;
  if (lc->magic == kShmListenMagic) {
    ShmListen* sl = (ShmListen*)listenComm;
    if (sl->link) link_unref(sl->link);   // never accepted: the object goes with it
    sl->magic = 0;
    delete sl;
    return ncclSuccess;
  }
  std::vector<Link*> orphans;
  {
    std::lock_guard<std::mutex> g(g_reg_mu);
    g_listens.erase(lc->id);
    orphans.assign(lc->pending.begin(), lc->pending.end());
  }
  for (Link* lk : orphans) {   // connects nobody will accept: tell the connecting side, drop the listener's share
    {
      std::lock_guard<ShortLock> g(lk->mu);
      lk->send_ready = -1;
    }
    link_unref(lk);
  }
  delete lc;
  return ncclSuccess;
}

// ---- v7 / v6 adapters ---------------------------------------------------------------------------------
ncclResult_t fl_get_properties_v7(int dev, ncclNetProperties_v7_t* p) {
  ncclNetProperties_v8_t q;
  ncclResult_t rc = fl_get_properties_v8(dev, &q);
  if (rc != ncclSuccess || !p) return rc != ncclSuccess ? rc : ncclInvalidArgument;
  p->name = q.name; p->pciPath = q.pciPath; p->guid = q.guid; p->ptrSupport = q.ptrSupport; p->speed = q.speed; p->port = q.port;
  p->latency = q.latency; p->maxComms = q.maxComms; p->maxRecvs = q.maxRecvs; p->netDeviceType = q.netDeviceType;
  p->netDeviceVersion = q.netDeviceVersion;
  return ncclSuccess;
}
ncclResult_t fl_get_properties_v6(int dev, ncclNetProperties_v6_t* p) {
  ncclNetProperties_v8_t q;
  ncclResult_t rc = fl_get_properties_v8(dev, &q);
  if (rc != ncclSuccess || !p) return rc != ncclSuccess ? rc : ncclInvalidArgument;
  p->name = q.name; p->pciPath = q.pciPath; p->guid = q.guid; p->ptrSupport = q.ptrSupport; p->speed = q.speed; p->port = q.port;
  p->latency = q.latency; p->maxComms = q.maxComms; p->maxRecvs = q.maxRecvs;
  return ncclSuccess;
}
ncclResult_t fl_reg_mr_v7(void* comm, void* data, int size, int type, void** mhandle) {
  if (size <= 0) return ncclInvalidArgument;
  return fl_reg_mr_dmabuf(comm, data, (size_t)size, type, 0ull, -1, mhandle);
}
ncclResult_t fl_connect_v7(int dev, void* handle, void** sendComm, ncclNetDeviceHandle_v7_t** d) { return fl_connect(dev, handle, sendComm, d); }
ncclResult_t fl_accept_v7(void* listenComm, void** recvComm, ncclNetDeviceHandle_v7_t** d) { return fl_accept(listenComm, recvComm, d); }
ncclResult_t fl_connect_v6(int dev, void* handle, void** sendComm) { return fl_connect(dev, handle, sendComm, nullptr); }
ncclResult_t fl_accept_v6(void* listenComm, void** recvComm) { return fl_accept(listenComm, recvComm, nullptr); }

}  // namespace

extern "C" {

__attribute__((visibility("default"))) ncclNet_v8_t ncclNetPlugin_v8 = {
    "FuseLink", fl_init, fl_devices, fl_get_properties_v8, fl_listen, fl_connect, fl_accept, fl_reg_mr_v8, fl_reg_mr_dmabuf,
    fl_dereg_mr, fl_isend, fl_irecv, fl_iflush, fl_test, fl_close_send, fl_close_recv, fl_close_listen,
    nullptr /* getDeviceMr */, nullptr /* irecvConsumed */};

__attribute__((visibility("default"))) ncclNet_v7_t ncclNetPlugin_v7 = {
    "FuseLink", fl_init, fl_devices, fl_get_properties_v7, fl_listen, fl_connect_v7, fl_accept_v7, fl_reg_mr_v7, fl_reg_mr_dmabuf,
    fl_dereg_mr, fl_isend, fl_irecv, fl_iflush, fl_test, fl_close_send, fl_close_recv, fl_close_listen,
    nullptr /* getDeviceMr */, nullptr /* irecvConsumed */};

__attribute__((visibility("default"))) ncclNet_v6_t ncclNetPlugin_v6 = {
    "FuseLink", fl_init, fl_devices, fl_get_properties_v6, fl_listen, fl_connect_v6, fl_accept_v6, fl_reg_mr_v7, fl_reg_mr_dmabuf,
    fl_dereg_mr, fl_isend, fl_irecv, fl_iflush, fl_test, fl_close_send, fl_close_recv, fl_close_listen};

int fl_net_set_credits(const uint32_t* credits, int n) {
  if (n < 0 || n > FL_NET_MAX_LANES || (n && !credits)) return fl_set_error(FLH_E_ARG, "bad credit row");
  std::lock_guard<std::mutex> g(g_credit_mu);
  g_credit_override = n > 0;
  for (int l = 0; l < FL_NET_MAX_LANES; ++l) g_credit_static[l] = l < n ? credits[l] : 0;
  return FLH_OK;
}

int fl_net_reset(void) {
  std::lock_guard<std::mutex> gi(g_init_mu);
  {
    std::lock_guard<std::mutex> g(g_reg_mu);
    if (!g_listens.empty() || g_live_links.load() != 0) return fl_set_error(FLH_E_STATE, "connections are still open");
  }
  {
    std::lock_guard<std::mutex> g(g_pool_mu);
    for (auto it = g_pools.begin(); it != g_pools.end(); it = g_pools.erase(it)) {
      int rc = flh_pool_destroy(it->second);
      if (rc < 0) return rc;
    }
  }
  g_par = Params();
  g_inited = false;
  for (auto& dir : g_last_mark) for (auto& cell : dir) cell.store(0, std::memory_order_relaxed);
  if (fl_monitor_is_shared()) fl_monitor_detach();  // back to the process-local table until init attaches again
  return FLH_OK;
}

int fl_net_inject_fault(void* request) {
  Request* r = (Request*)request;
  if (!r || r->magic != kReqMagic || r->type == kReqUnused) return fl_set_error(FLH_E_ARG, "not a request in flight");
  std::lock_guard<ShortLock> g(r->link->mu);
  r->fault = 1;
  return FLH_OK;
}

int fl_net_comm_stats(void* comm, int64_t* n_finished, int64_t* in_flight, int64_t* refreshes) {
  Comm* c = (Comm*)comm;
  if (!c || c->magic != kCommMagic) return fl_set_error(FLH_E_ARG, "not a send or recv comm");
  Link* lk = c->link;
  std::lock_guard<ShortLock> g(lk->mu);
  if (n_finished) *n_finished = c->is_send ? lk->s_finished : lk->r_finished;
  if (in_flight) *in_flight = c->is_send ? lk->s_inflight : lk->r_inflight;
  if (refreshes) *refreshes = lk->refreshes;
  return FLH_OK;
}

int fl_net_mask_stats(void* comm, uint32_t* mask, int64_t* refreshes) {
  Comm* c = (Comm*)comm;
  if (!c || c->magic != kCommMagic) return fl_set_error(FLH_E_ARG, "not a send or recv comm");
  Link* lk = c->link;
  std::lock_guard<ShortLock> g(lk->mu);
  if (mask) *mask = c->is_send ? lk->tx_mask : lk->tx_available;
  if (refreshes) *refreshes = c->is_send ? lk->tx_refreshes : lk->refreshes;
  return FLH_OK;
}

int fl_net_free_requests(void* comm) {
  Comm* c = (Comm*)comm;
  if (!c || c->magic != kCommMagic) return fl_set_error(FLH_E_ARG, "not a send or recv comm");
  Link* lk = c->link;
  std::lock_guard<ShortLock> g(lk->mu);
  const Request* tab = c->is_send ? lk->sreq : lk->rreq;
  int n = 0;
  for (int i = 0; i < FL_NET_MAX_REQUESTS; ++i) n += tab[i].type == kReqUnused;
  return n;
}

int fl_net_launch_stats(void* comm, int64_t* launches, int64_t* batched_requests) {
  Comm* c = (Comm*)comm;
  if (!c || c->magic != kCommMagic) return fl_set_error(FLH_E_ARG, "not a send or recv comm");
  Link* lk = c->link;
  Peer* pr = lk->peer.load(std::memory_order_acquire);
  if (!pr) {
    if (launches) *launches = 0;
    if (batched_requests) *batched_requests = 0;
    return FLH_OK;
  }
  std::lock_guard<std::mutex> g(pr->launch_mu);
  if (launches) *launches = lk->launches;
  if (batched_requests) *batched_requests = lk->batched_requests;
  return FLH_OK;
}

// launch everything that waits and wait for the stream (launch_mu held)
static int drain_peer(Peer* pr) {
  flush_pending(pr);
  DeviceScope keep;
  if (hipSetDevice(pr->hip_device) != hipSuccess || hipStreamSynchronize(pr->stream) != hipSuccess) return fl_set_error(FLH_E_HIP, "stream synchronize failed");
  if (pr->engine) {
    const int64_t until = tr_now() + 5000000000ll;
    while (flh_engine_completed(pr->engine) < pr->engine_submitted.load(std::memory_order_acquire)) {
      if (flh_engine_error(pr->engine) || tr_now() > until) return fl_set_error(FLH_E_STATE, "the lane engine did not finish its batches");
      if (flh_engine_needs_start(pr->engine)) (void)flh_engine_poke(pr->engine);
    }
  }
  return FLH_OK;
}

// table and header of the peer's last launch or engine batch (launch_mu held, the peer drained)
static void last_buffers(const Peer* pr, const flh_chunk_desc** table, const flh_sched_hdr** hdr) {
  if (pr->last.engine) {
    const uint32_t slot = (uint32_t)((pr->last.seq - 1) % kEngineSlots);
    *table = pr->d_etable + (size_t)slot * kEngineRows;
    *hdr = pr->d_ehdr + slot;
  } else {
    *table = pr->d_table;
    *hdr = pr->d_hdr;
  }
}

int fl_net_last_table(void* sendComm, void* rows_out, int max_rows, void* hdr_out) {
  Comm* c = (Comm*)sendComm;
  if (!c || c->magic != kCommMagic || !c->is_send) return fl_set_error(FLH_E_ARG, "not a send comm");
  Link* lk = c->link;
  Peer* pr = lk->peer.load(std::memory_order_acquire);
  if (!pr) return fl_set_error(FLH_E_STATE, "the connection has not staged anything yet");
  std::lock_guard<std::mutex> gl(pr->launch_mu);
  int rc = drain_peer(pr);
  if (rc) return rc;
  if (lk->last_seq == 0) return fl_set_error(FLH_E_STATE, "the connection has not staged anything yet");
  if (lk->last_seq != pr->last.seq || lk->last_engine != pr->last.engine) return fl_set_error(FLH_E_STATE, "a later launch of another connection has reused the table");
  const int rows = (int)lk->last_rows;
  const int take = rows < max_rows ? rows : max_rows;
  const flh_chunk_desc* table;
  const flh_sched_hdr* hdr;
  last_buffers(pr, &table, &hdr);
  DeviceScope keep;
  if (hipSetDevice(pr->hip_device) != hipSuccess) return fl_set_error(FLH_E_HIP, "hipSetDevice failed");
  if (take > 0 && rows_out && hipMemcpy(rows_out, table + lk->last_first_row, sizeof(flh_chunk_desc) * (size_t)take, hipMemcpyDeviceToHost) != hipSuccess)
    return fl_set_error(FLH_E_HIP, "table copy failed");
  if (hdr_out && hipMemcpy(hdr_out, hdr, sizeof(flh_sched_hdr), hipMemcpyDeviceToHost) != hipSuccess)
    return fl_set_error(FLH_E_HIP, "header copy failed");
  return rows;
}

int fl_net_last_launch(void* comm, fl_net_launch_seg* segs_out, int max_segs, void* rows_out, int max_rows, void* hdr_out) {
  Comm* c = (Comm*)comm;
  if (!c || c->magic != kCommMagic) return fl_set_error(FLH_E_ARG, "not a send or recv comm");
  Peer* pr = c->link->peer.load(std::memory_order_acquire);
  if (!pr) return fl_set_error(FLH_E_STATE, "the connection has not staged anything yet");
  std::lock_guard<std::mutex> gl(pr->launch_mu);
  int rc = drain_peer(pr);
  if (rc) return rc;
  const LaunchInfo& li = pr->last;
  for (int k = 0; k < (int)li.n_seg && k < max_segs && segs_out; ++k) {
    fl_net_launch_seg& o = segs_out[k];
    o.channel = li.seg[k].channelId;
    o.first_row = li.seg[k].first_row;
    o.n_rows = li.seg[k].n_rows;
    o.n_req = li.seg[k].n_req;
    o.epoch_bytes = li.seg[k].epoch_bytes;
    for (int l = 0; l < FL_NET_MAX_LANES; ++l) o.lane_base[l] = li.seg[k].lane_base[l];
  }
  const int take = (int)li.n_rows < max_rows ? (int)li.n_rows : max_rows;
  const flh_chunk_desc* table;
  const flh_sched_hdr* hdr;
  last_buffers(pr, &table, &hdr);
  DeviceScope keep;
  if (hipSetDevice(pr->hip_device) != hipSuccess) return fl_set_error(FLH_E_HIP, "hipSetDevice failed");
  if (take > 0 && rows_out && hipMemcpy(rows_out, table, sizeof(flh_chunk_desc) * (size_t)take, hipMemcpyDeviceToHost) != hipSuccess)
    return fl_set_error(FLH_E_HIP, "table copy failed");
  if (hdr_out && hipMemcpy(hdr_out, hdr, sizeof(flh_sched_hdr), hipMemcpyDeviceToHost) != hipSuccess)
    return fl_set_error(FLH_E_HIP, "header copy failed");
  return (int)li.n_seg;
}

int fl_net_host_stats(int64_t* calls_out, int64_t* ns_out, int n) {
  std::lock_guard<std::mutex> g(g_tr_mu);
  for (int k = 0; k < n && k < kTrCount; ++k) {
    int64_t calls = 0, ns = 0;
    for (const TraceCounters* t : g_tr_blocks) { calls += t->calls[k].load(std::memory_order_relaxed); ns += t->ns[k].load(std::memory_order_relaxed); }
    if (calls_out) calls_out[k] = calls;
    if (ns_out) ns_out[k] = ns;
  }
  return kTrCount;
}

int fl_net_timeline(void* out, int max_events) {
  const uint64_t n = g_timeline_n.load(std::memory_order_acquire);
  const uint64_t have = n < kTimelineCap ? n : kTimelineCap;
  const uint64_t take = have < (uint64_t)(max_events > 0 ? max_events : 0) ? have : (uint64_t)(max_events > 0 ? max_events : 0);
  if (out && take) memcpy(out, g_timeline, take * sizeof(TimelineEvent));
  return (int)have;
}

int fl_net_flush(void* comm) {
  Comm* c = (Comm*)comm;
  if (!c || c->magic != kCommMagic) return fl_set_error(FLH_E_ARG, "not a send or recv comm");
  Peer* pr = c->link->peer.load(std::memory_order_acquire);
  if (!pr) return FLH_OK;
  std::lock_guard<std::mutex> gl(pr->launch_mu);
  flush_pending(pr);
  return FLH_OK;
}

}  // extern "C"
