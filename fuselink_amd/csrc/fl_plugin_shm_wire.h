// fl_plugin_shm_wire.h -- the plugin's wire between two processes.  Not a header of its own: fl_plugin.cc includes it
// inside its unnamed namespace, behind the objects and helpers it uses (Params, FifoWire, Link, Peer, Request, Handle,
// DeviceScope, FL_HIPCHECK / FL_FLHCHECK, ensure_pool, attach_peer, wire_credits, fill_uniform, the completion helpers)
// and in front of the entry points that dispatch to it.
// ------------------------------------------------------------------------------------------------
// shared-memory wire: sender and receiver in different processes (NCCL_FUSELINK_WIRE=shm)
// ------------------------------------------------------------------------------------------------
// The reference's two ends are different processes on different hosts: the receiver writes 64-byte descriptors into a
// FIFO in the sender's memory by RDMA (ncclIbSendFifo, plugin.cc:487-496, 1616-1677), the sender RDMA-writes the payload
// out of its staged buffer into the receiver's registered memory and completes it with a WRITE_WITH_IMM whose immediate
// data is its lane-availability mask (plugin.cc:1441-1465, 1467-1495), and the 128-byte handle that listen fills carries
// what connect needs to reach the listener (plugin.cc:425-430, 776-885).  On one GPU the part of that which can be shown
// is the process boundary.
//
// Per connection: listen creates a POSIX shared-memory object and names it in the handle; connect, in another process,
// maps it.  It holds the descriptor FIFO (receiver writes, sender reads).
// Per pair of processes and GPU: the receiver owns sets of landing windows, one window per lane in each set, device
// memory that the sender opens through hipIpcOpenMemHandle (an imported VMM allocation would be the closer analogue;
// this runtime refuses hipMemImportFromShareableHandle for another process's descriptor), and a second shared-memory
// object with a ring of wave records -- the stand-in for the WRITE_WITH_IMM completions -- shared by every connection
// between the two processes, as the reference's channels share the per-NIC lane comms (fuselink.h:271-272).
//
// A send travels through the sending GPU's staging side like a send whose receiver is in the same process
// (fl_plugin.cc): matched sends of all connections wait in one queue and go out in batches.  A batch for another
// process is a *wave*: the lane engine (or, for large requests, one launch) stripes it into this process's staging
// windows and carries every staged tile on into the same lane and offset of one set of landing windows
// (FLH_ENGINE_SEND / flh_stripe_*_carry: the NIC's part).  When the engine's completion word -- or the launch's --
// says the bytes have landed, the sender's test publishes the wave record from the host and reports the sends complete:
// like an RDMA write, a send is complete once its bytes are in the receiver's memory.  The receiver's test finds the
// record, builds the same batch from the receives it posted (it wrote their credit rows into the descriptors itself;
// the record brings the sizes, the epoch prefixes and the sender's masks) and hands it to its own engine
// (FLH_ENGINE_RECV) or launches the reassembly; when that is complete the landing set goes back to the sender through a
// counter.  No event is recorded or queried and, for requests the engine takes, nothing is launched on either side.

constexpr uint64_t kHandleMagicShm = 0x4655534c53484d32ull;   // "FUSLSHM2"
constexpr uint64_t kPairMagic = 0x4655534c50414952ull;        // "FUSLPAIR"
constexpr uint32_t kShmListenMagic = 0x464c534c;              // "FLSL"

constexpr int kShmSetsMax = 8;
constexpr uint32_t kPairWaves = 64;      // wave records a pair's ring holds (more than the landing sets there can be)
constexpr uint32_t kPairConns = 256;     // connections between two processes that share the pair
constexpr uint32_t kPairMrs = 64;        // registrations of the receiver that the sender can write into directly
// Every wave, whichever way it travels, is numbered only while fewer than `sets` waves are unconsumed (wire_set_free), so
// a record of the ring is never written again before the receiver has taken it.
static_assert(kPairWaves > (uint32_t)kShmSetsMax, "the ring of wave records must hold every wave that can be unconsumed");

struct WaveReq {                   // one request of a wave
  uint32_t conn;                   // the connection's number within the pair
  uint32_t imm;                    // the sender's lane-availability mask: imm_data of plugin.cc:1441-1447, 1463
  uint64_t fifo_idx;               // the descriptor it answers, from 1
  uint64_t bytes;
};
struct WaveSeg {                   // a run of requests of one connection, scheduled as one message (flh_batch_segment)
  uint64_t epoch_bytes;            // the connection's credit-epoch prefix the segment was scheduled from
  uint32_t n_req;
  uint32_t pad;
};
struct ShmWave {                   // one wave that has landed in the receiver's windows
  std::atomic<uint64_t> seq;       // wave number (from 1), written last
  uint32_t set;                    // the set of landing windows it lies in
  uint32_t n_req, n_seg;
  uint32_t piece;                  // 1: part of ONE request that the windows do not hold whole: `offset` and `last` apply
  uint64_t offset;                 // byte offset of the piece in the request
  uint32_t last;                   // the request's last piece
  uint32_t direct;                 // 1: the bytes are already in the posted buffers (written through the registrations' rkeys): nothing to deliver
  uint64_t total_bytes;
  WaveReq req[FLH_BATCH_MAX];
  WaveSeg seg[FLH_SEG_MAX];
};
// A registration of the receiver that the sender may write into directly, as an RDMA write lands in the receiver's
// registered memory (plugin.cc:1485-1486: remote_addr and rkey come from the descriptor): the whole allocation around
// the registered buffer, exported through HIP IPC.  The descriptor's rkey names the entry and its generation.
struct ShmMr {
  std::atomic<uint32_t> gen;       // odd while the registration stands; moves on when it goes
  uint32_t pad;
  uint64_t base, size;             // in the receiver's address space
  hipIpcMemHandle_t handle;
};
struct ShmPair {                   // one per (sending process, receiving process, GPU of the receiver)
  uint64_t magic;
  uint32_t lanes;
  uint32_t sets;                   // sets of landing windows = waves that may be on the wire at once
  uint64_t bytes_per_lane;
  hipIpcMemHandle_t landing;       // sets x lanes x bytes_per_lane of the receiver's device memory
  std::atomic<uint32_t> sender_mapped;   // the sender holds its mapping: the name is no longer needed
  std::atomic<uint32_t> failed;          // a wave was lost (the sender's engine went down): every request on the pair fails
  alignas(64) std::atomic<uint64_t> waves_consumed;   // receiver: waves delivered so far, in order (their landing sets are free again)
  alignas(64) ShmMr mr[kPairMrs];
  alignas(64) ShmWave wave[kPairWaves];
};
struct ShmWire {                   // one per connection
  uint64_t magic;
  uint32_t lanes;
  uint32_t channelId;
  std::atomic<uint32_t> connected, accepted, send_closed, recv_closed;
  int32_t sender_pid;              // written by connect
  std::atomic<uint32_t> landing_ready;   // pair_name and pair_conn are valid
  uint32_t pair_conn;
  char pair_name[64];
  alignas(64) FifoWire fifo[FL_NET_MAX_REQUESTS];   // plugin.cc:487-496: written by the receiver, idx last; cleared by the sender when matched
};

struct WireFlight {                // a wave whose GPU work has been handed over
  bool engine = false;
  uint64_t seq = 0;                // engine batch or launch that completes it (0: no GPU work, complete as it stands)
  ShmWave rec;                     // sender: the record to publish
  WireFlight() { memset((void*)&rec, 0, sizeof(rec)); }
  WireFlight(const WireFlight& o) : engine(o.engine), seq(o.seq) { memcpy((void*)&rec, (const void*)&o.rec, sizeof(rec)); }
  WireFlight& operator=(const WireFlight&) = delete;
};

struct WirePair {                  // this process's end of a pair
  ShmPair* w = nullptr;
  char name[64] = "";
  bool receiver = false;           // this process owns the landing windows and the object
  bool named = false;              // the name still exists in the file system
  int peer_pid = 0;
  int hip_device = -1;
  int links = 0;                   // connections attached (g_pair_mu)
  Peer* peer = nullptr;            // this process's staging side of the GPU
  uint8_t* landing = nullptr;      // receiver: its allocation; sender: the same memory opened through IPC
  int sets = 0;
  flh_windows landing_wins[kShmSetsMax] = {};
  // sender (flights and tx_launched under tx_mu)
  std::mutex tx_mu;
  std::deque<WireFlight> tx_flights;
  uint64_t tx_launched = 0;                     // waves handed to the GPU
  std::atomic<uint64_t> tx_published{0};        // waves announced to the receiver
  bool blocked = false;                         // a pass that launches found no free landing set (launch_mu)
  // receiver (under rx_mu)
  std::mutex rx_mu;
  std::deque<WireFlight> rx_flights;
  std::atomic<uint64_t> rx_taken{0};            // waves taken off the ring
  uint64_t rx_done = 0;                         // waves delivered
  std::atomic<Link*> conns[kPairConns] = {};    // this process's end of every connection of the pair, by its number
  // registrations that can be written directly (mr_mu): the receiver's reference counts by allocation, the sender's mappings
  std::mutex mr_mu;
  struct { uint64_t base; int refs; } mr_local[kPairMrs] = {};
  struct { uint8_t* ptr; uint32_t gen; uint64_t base, size; } mr_map[kPairMrs] = {};
};

struct WireEnd {                   // a connection's end of the wire (Link::wire)
  ShmWire* w = nullptr;
  char name[64] = "";
  bool owner = false;              // the receiver created the object and unlinks it
  bool is_send = false;
  WirePair* pair = nullptr;
  uint32_t pair_conn = 0;
};

struct ShmListen {
  uint32_t magic = kShmListenMagic;
  int dev = 0;
  Link* link = nullptr;            // becomes the recv comm's at accept
};

std::atomic<uint64_t> g_shm_counter{0};
std::mutex g_pair_mu;              // the pairs of this process, their attachment counts and connection tables
std::vector<WirePair*> g_pairs;

void wire_pair_destroy(WirePair* p) {   // no longer reachable through g_pairs
  for (auto& m : p->mr_map) {
    if (!m.ptr) continue;
    DeviceScope keep;
    (void)hipSetDevice(p->hip_device);
    (void)hipIpcCloseMemHandle(m.ptr);
    m.ptr = nullptr;
  }
  if (p->landing) {
    DeviceScope keep;
    (void)hipSetDevice(p->hip_device);
    if (p->receiver) {
      // what this process's kernels still read out of the windows must be through before they go
      if (p->peer && p->peer->stream) (void)hipStreamSynchronize(p->peer->stream);
      (void)hipFree(p->landing);
    } else {
      (void)hipIpcCloseMemHandle(p->landing);
    }
  }
  if (p->w) munmap(p->w, sizeof(ShmPair));
  if (p->receiver && p->named) shm_unlink(p->name);
  delete p;
}

// The connection's end goes away (the last reference to the link is being dropped; nothing of it waits for a launch).
void wire_end_free(Link* lk) {
  WireEnd* e = lk->wire;
  if (!e) return;
  if (e->w) (e->is_send ? e->w->send_closed : e->w->recv_closed).store(1, std::memory_order_release);
  if (WirePair* p = e->pair) {
    bool gone;
    {
      std::lock_guard<std::mutex> g(g_pair_mu);
      if (p->receiver) p->conns[e->pair_conn].store(nullptr, std::memory_order_release);
      gone = --p->links == 0;
      if (gone) {
        for (size_t i = 0; i < g_pairs.size(); ++i) if (g_pairs[i] == p) { g_pairs.erase(g_pairs.begin() + (long)i); break; }
      }
    }
    if (gone) wire_pair_destroy(p);
  }
  if (e->w) munmap(e->w, sizeof(ShmWire));
  if (e->owner && e->name[0]) shm_unlink(e->name);
  delete e;
  lk->wire = nullptr;
}

ncclResult_t shm_listen(int dev, void* opaqueHandle, void** listenComm) {
  ShmListen* lc = new (std::nothrow) ShmListen();
  Link* lk = new (std::nothrow) Link();
  WireEnd* e = new (std::nothrow) WireEnd();
  if (!lc || !lk || !e) { delete lc; delete lk; delete e; return ncclSystemError; }
  snprintf(e->name, sizeof(e->name), "/fuselink-wire-%d-%llu", (int)getpid(), (unsigned long long)g_shm_counter.fetch_add(1));
  int fd = shm_open(e->name, O_CREAT | O_EXCL | O_RDWR, 0600);
  if (fd < 0 || ftruncate(fd, sizeof(ShmWire)) != 0) { if (fd >= 0) { close(fd); shm_unlink(e->name); } FL_WARN("NET/FuseLink : shm_open(%s) failed", e->name); delete lc; delete lk; delete e; return ncclSystemError; }
  void* p = mmap(nullptr, sizeof(ShmWire), PROT_READ | PROT_WRITE, MAP_SHARED, fd, 0);
  close(fd);
  if (p == MAP_FAILED) { shm_unlink(e->name); delete lc; delete lk; delete e; return ncclSystemError; }
  memset(p, 0, sizeof(ShmWire));
  g_live_links.fetch_add(1);
  e->w = (ShmWire*)p;
  e->owner = true;
  e->is_send = false;
  e->w->lanes = (uint32_t)g_par.lanes;
  {
    std::lock_guard<std::mutex> g(g_reg_mu);
    e->w->channelId = (uint32_t)g_channel_counter++;
  }
  e->w->magic = kHandleMagicShm;
  lk->refs = 1;
  lk->dev = dev;
  lk->channelId = (int)e->w->channelId;
  lk->send_ready = 1;
  lk->wire = e;
  lc->dev = dev;
  lc->link = lk;
  Handle* h = (Handle*)opaqueHandle;
  memset(h, 0, NCCL_NET_HANDLE_MAXSIZE);
  h->magic = kHandleMagicShm;
  h->channelId = (int32_t)e->w->channelId;
  h->dev = dev;
  // the object's name travels in the handle, as the listener's address does in the reference's (plugin.cc:425-430)
  static_assert(sizeof(Handle) + 64 <= NCCL_NET_HANDLE_MAXSIZE, "the name must fit behind the fixed part of the handle");
  memcpy((char*)opaqueHandle + sizeof(Handle), e->name, sizeof(e->name));
  *listenComm = lc;
  return ncclSuccess;
}

ncclResult_t shm_connect(int dev, void* opaqueHandle, void** sendComm) {
  Handle* h = (Handle*)opaqueHandle;
  *sendComm = nullptr;
  Link* lk = (Link*)h->stage_link;
  if (h->stage == 0) {
    char name[64];
    memcpy(name, (char*)opaqueHandle + sizeof(Handle), sizeof(name));
    name[63] = 0;
    int fd = shm_open(name, O_RDWR, 0600);
    if (fd < 0) { FL_WARN("NET/FuseLink : connect: no shared-memory object %s (is the listener alive?)", name); return ncclSystemError; }
    // the object is the other process's: it must be the size this build gives the wire (a listener of another build
    // lays it out differently, and touching pages beyond a shorter object would raise SIGBUS)
    struct stat st;
    if (fstat(fd, &st) != 0 || (size_t)st.st_size != sizeof(ShmWire)) {
      FL_WARN("NET/FuseLink : connect: the shared-memory object %s holds %lld bytes, this build's wire %zu: the listener runs another build", name,
              (long long)st.st_size, sizeof(ShmWire));
      close(fd);
      return ncclInvalidUsage;
    }
    void* p = mmap(nullptr, sizeof(ShmWire), PROT_READ | PROT_WRITE, MAP_SHARED, fd, 0);
    close(fd);
    if (p == MAP_FAILED) return ncclSystemError;
    lk = new (std::nothrow) Link();
    WireEnd* e = new (std::nothrow) WireEnd();
    if (!lk || !e) { delete lk; delete e; munmap(p, sizeof(ShmWire)); return ncclSystemError; }
    g_live_links.fetch_add(1);
    e->w = (ShmWire*)p;
    e->is_send = true;
    memcpy(e->name, name, sizeof(name));
    lk->refs = 1;
    lk->dev = dev;
    lk->channelId = (int)e->w->channelId;
    lk->send_ready = 1;
    lk->wire = e;
    if (e->w->magic != kHandleMagicShm || (int)e->w->lanes != g_par.lanes) {
      FL_WARN("NET/FuseLink : connect: the listener runs %u lanes, this side %d", e->w->lanes, g_par.lanes);
      e->w = nullptr;               // not ours to mark closed
      munmap(p, sizeof(ShmWire));
      link_unref(lk);
      return ncclInvalidUsage;
    }
    int listener_pid = -1;
    if (sscanf(name, "/fuselink-wire-%d-", &listener_pid) == 1 && listener_pid == (int)getpid()) {
      // the landing windows reach the sender through HIP IPC, which a process cannot open on its own allocations
      FL_WARN("NET/FuseLink : NCCL_FUSELINK_WIRE=shm connects two processes; this listener lives in the connecting process (unset it for the in-process wire)");
      e->w = nullptr;
      munmap(p, sizeof(ShmWire));
      link_unref(lk);
      return ncclInvalidUsage;
    }
    e->w->sender_pid = (int32_t)getpid();
    e->w->connected.store(1, std::memory_order_release);
    h->stage = 1;
    h->stage_link = lk;
    return ncclSuccess;
  }
  if (!lk->wire->w->accepted.load(std::memory_order_acquire)) return ncclSuccess;   // accept has not happened yet
  Comm* c = new (std::nothrow) Comm();
  if (!c) return ncclSystemError;
  c->is_send = 1;
  c->link = lk;
  h->stage = 0;
  h->stage_link = nullptr;
  *sendComm = c;
  return ncclSuccess;
}

ncclResult_t shm_accept(ShmListen* lc, void** recvComm) {
  *recvComm = nullptr;
  Link* lk = lc->link;
  if (!lk || !lk->wire->w->connected.load(std::memory_order_acquire)) return ncclSuccess;   // nobody connected yet
  Comm* c = new (std::nothrow) Comm();
  if (!c) return ncclSystemError;
  WireEnd* e = lk->wire;
  e->w->accepted.store(1, std::memory_order_release);
  shm_unlink(e->name);   // both ends hold their mapping: the name is no longer needed and cannot leak
  e->owner = false;
  lc->link = nullptr;
  c->is_send = 0;
  c->link = lk;
  *recvComm = c;
  return ncclSuccess;
}

// set k, lane l of the landing windows: one allocation, set after set, lane after lane
void wire_landing_windows(WirePair* p, uint64_t per_lane) {
  for (int k = 0; k < p->sets; ++k) {
    p->landing_wins[k].n_lanes = (uint32_t)g_par.lanes;
    for (int l = 0; l < g_par.lanes; ++l) {
      p->landing_wins[k].base[l] = p->landing + ((uint64_t)k * (uint64_t)g_par.lanes + (uint64_t)l) * per_lane;
      p->landing_wins[k].cap[l] = per_lane;
    }
  }
}

// what a window of either kind (the launches', the engine's) holds in this process
uint64_t wire_window_cap() {
  const uint64_t a = (uint64_t)g_par.window_units * FLH_UNIT_BYTES, b = g_par.engine ? (uint64_t)g_par.engine_units * FLH_UNIT_BYTES : 0;
  return a > b ? a : b;
}

// Receiver (lk->mu held): the connection joins the pair of its sender's process and this GPU -- the first one creates
// it, landing windows and all -- and tells the sender where to find it.
ncclResult_t wire_recv_setup(Link* lk, int device) {
  WireEnd* e = lk->wire;
  if (e->pair) return ncclSuccess;
  ncclResult_t rc = attach_peer(lk, device);   // this process's staging side of the GPU: engine, stream, completion words
  if (rc != ncclSuccess) return rc;
  const int sender = (int)e->w->sender_pid;
  std::lock_guard<std::mutex> g(g_pair_mu);
  WirePair* p = nullptr;
  for (WirePair* q : g_pairs) if (q->receiver && q->peer_pid == sender && q->hip_device == device) { p = q; break; }
  if (!p) {
    p = new (std::nothrow) WirePair();
    if (!p) return ncclSystemError;
    p->receiver = true;
    p->peer_pid = sender;
    p->hip_device = device;
    p->peer = lk->peer.load(std::memory_order_acquire);
    snprintf(p->name, sizeof(p->name), "/fuselink-pair-%d-%d-%d-%llu", (int)getpid(), sender, device, (unsigned long long)g_shm_counter.fetch_add(1));
    int fd = shm_open(p->name, O_CREAT | O_EXCL | O_RDWR, 0600);
    if (fd < 0 || ftruncate(fd, sizeof(ShmPair)) != 0) { if (fd >= 0) { close(fd); shm_unlink(p->name); } FL_WARN("NET/FuseLink : shm_open(%s) failed", p->name); delete p; return ncclSystemError; }
    void* m = mmap(nullptr, sizeof(ShmPair), PROT_READ | PROT_WRITE, MAP_SHARED, fd, 0);
    close(fd);
    if (m == MAP_FAILED) { shm_unlink(p->name); delete p; return ncclSystemError; }
    memset(m, 0, sizeof(ShmPair));
    p->w = (ShmPair*)m;
    p->named = true;
    const uint64_t cap = wire_window_cap();
    p->sets = g_par.wire_sets;
    while (p->sets > 1 && cap * (uint64_t)g_par.lanes * (uint64_t)p->sets >= (2ull << 30)) p->sets--;   // a shared allocation must stay under 2 GiB
    const uint64_t bytes = cap * (uint64_t)g_par.lanes * (uint64_t)p->sets;
    DeviceScope keep;
    hipError_t he = bytes >= (2ull << 30) ? hipErrorInvalidValue : hipSetDevice(device);
    if (he == hipSuccess) he = hipMalloc((void**)&p->landing, bytes);
    if (he == hipSuccess) he = hipIpcGetMemHandle(&p->w->landing, p->landing);
    if (he != hipSuccess) {
      FL_WARN("NET/FuseLink : %d sets of landing windows (%llu bytes): %s", p->sets, (unsigned long long)bytes, bytes >= (2ull << 30) ? "a shared allocation must stay under 2 GiB" : hipGetErrorString(he));
      wire_pair_destroy(p);
      return bytes >= (2ull << 30) ? ncclInvalidUsage : ncclUnhandledCudaError;
    }
    p->w->lanes = (uint32_t)g_par.lanes;
    p->w->sets = (uint32_t)p->sets;
    p->w->bytes_per_lane = cap;
    p->w->magic = kPairMagic;
    wire_landing_windows(p, cap);
    g_pairs.push_back(p);
  }
  uint32_t id = kPairConns;
  for (uint32_t i = 0; i < kPairConns && id == kPairConns; ++i) {
    Link* none = nullptr;
    if (p->conns[i].compare_exchange_strong(none, lk, std::memory_order_acq_rel)) id = i;
  }
  if (id == kPairConns) { FL_WARN("NET/FuseLink : more than %u connections between two processes", kPairConns); if (p->links == 0) { g_pairs.pop_back(); wire_pair_destroy(p); } return ncclInternalError; }
  p->links++;
  e->pair = p;
  e->pair_conn = id;
  memcpy(e->w->pair_name, p->name, sizeof(p->name));
  e->w->pair_conn = id;
  e->w->landing_ready.store(1, std::memory_order_release);
  return ncclSuccess;
}

// Sender (lk->mu held): opens the pair the receiver announced.  *ready stays false while the receiver has not got that far.
ncclResult_t wire_send_setup(Link* lk, int device, bool* ready) {
  WireEnd* e = lk->wire;
  *ready = e->pair != nullptr;
  if (*ready) return ncclSuccess;
  if (!e->w->landing_ready.load(std::memory_order_acquire)) return ncclSuccess;
  ncclResult_t rc = attach_peer(lk, device);
  if (rc != ncclSuccess) return rc;
  char name[64];
  memcpy(name, e->w->pair_name, sizeof(name));
  name[63] = 0;
  std::lock_guard<std::mutex> g(g_pair_mu);
  WirePair* p = nullptr;
  for (WirePair* q : g_pairs) if (!q->receiver && !strcmp(q->name, name)) { p = q; break; }
  if (!p) {
    int fd = shm_open(name, O_RDWR, 0600);
    struct stat st;
    if (fd < 0 || fstat(fd, &st) != 0 || (size_t)st.st_size != sizeof(ShmPair)) {
      if (fd >= 0) close(fd);
      FL_WARN("NET/FuseLink : the receiver's landing windows (%s) cannot be reached, or belong to another build", name);
      return ncclSystemError;
    }
    void* m = mmap(nullptr, sizeof(ShmPair), PROT_READ | PROT_WRITE, MAP_SHARED, fd, 0);
    close(fd);
    if (m == MAP_FAILED) return ncclSystemError;
    p = new (std::nothrow) WirePair();
    if (!p) { munmap(m, sizeof(ShmPair)); return ncclSystemError; }
    p->w = (ShmPair*)m;
    memcpy(p->name, name, sizeof(name));
    p->hip_device = device;
    p->peer = lk->peer.load(std::memory_order_acquire);
    if (p->w->magic != kPairMagic || (int)p->w->lanes != g_par.lanes || p->w->sets < 1 || p->w->sets > (uint32_t)kShmSetsMax || p->w->bytes_per_lane < wire_window_cap()) {
      FL_WARN("NET/FuseLink : the receiver's landing windows (%u sets of %llu bytes per lane, %u lanes) do not fit this side's staging windows (%llu bytes, %d lanes)",
              p->w->sets, (unsigned long long)p->w->bytes_per_lane, p->w->lanes, (unsigned long long)wire_window_cap(), g_par.lanes);
      wire_pair_destroy(p);
      return ncclInvalidUsage;
    }
    DeviceScope keep;
    hipError_t he = hipSetDevice(device);
    if (he == hipSuccess) he = hipIpcOpenMemHandle((void**)&p->landing, p->w->landing, hipIpcMemLazyEnablePeerAccess);
    if (he != hipSuccess) { p->landing = nullptr; wire_pair_destroy(p); return hip_fail("hipIpcOpenMemHandle", he); }
    p->sets = (int)p->w->sets;
    wire_landing_windows(p, p->w->bytes_per_lane);
    p->w->sender_mapped.store(1, std::memory_order_release);
    g_pairs.push_back(p);
  }
  p->links++;
  e->pair = p;
  e->pair_conn = e->w->pair_conn;
  *ready = true;
  return ncclSuccess;
}

// ---- registrations the sender writes into directly --------------------------------------------------------------------
bool wire_pair_alive(WirePair* p) {   // g_pair_mu held
  for (WirePair* q : g_pairs) if (q == p) return true;
  return false;
}
// Receiver, at regMr: export the allocation [base, base + bytes) to the pair's sender.  *rkey stays 0 when that is not
// possible (switched off, 2 GiB or more -- what HIP IPC carries reliably here --, memory the runtime cannot export, table
// full): such a buffer is reached through the landing windows instead.
void wire_export_mr(WirePair* p, void* base, size_t bytes, uint32_t* rkey) {
  *rkey = 0;
  if (!g_par.wire_direct || bytes >= (2ull << 30)) return;
  std::lock_guard<std::mutex> g(p->mr_mu);
  int at = -1;
  for (uint32_t i = 0; i < kPairMrs; ++i) {
    if (p->mr_local[i].refs > 0 && p->mr_local[i].base == (uint64_t)(uintptr_t)base && p->w->mr[i].size == bytes) {
      p->mr_local[i].refs++;
      *rkey = ((p->w->mr[i].gen.load(std::memory_order_relaxed) & 0xffffffu) << 8) | (i + 1);
      return;
    }
    if (at < 0 && p->mr_local[i].refs == 0) at = (int)i;
  }
  if (at < 0) return;
  ShmMr& m = p->w->mr[at];
  DeviceScope keep;
  if (hipSetDevice(p->hip_device) != hipSuccess || hipIpcGetMemHandle(&m.handle, base) != hipSuccess) {
    (void)hipGetLastError();   // not an error of the registration: the landing windows carry it
    return;
  }
  m.base = (uint64_t)(uintptr_t)base;
  m.size = bytes;
  const uint32_t old = m.gen.load(std::memory_order_relaxed);
  const uint32_t gen = (old & 1u) ? old + 2 : old + 1;
  m.gen.store(gen, std::memory_order_release);   // odd: the entry stands
  p->mr_local[at].base = m.base;
  p->mr_local[at].refs = 1;
  *rkey = ((gen & 0xffffffu) << 8) | ((uint32_t)at + 1);
}
void wire_unexport_mr(WirePair* p, uint32_t rkey) {
  std::lock_guard<std::mutex> ga(g_pair_mu);
  if (!wire_pair_alive(p)) return;   // the pair went with its last connection, and the table with it
  const uint32_t i = (rkey & 0xffu) - 1;
  if (i >= kPairMrs) return;
  std::lock_guard<std::mutex> g(p->mr_mu);
  if (p->mr_local[i].refs > 0 && --p->mr_local[i].refs == 0) p->w->mr[i].gen.fetch_add(1, std::memory_order_release);   // even: gone
}
// Sender: where `bytes` at the receiver's address `addr` lie in this process, through the registration `rkey` names;
// null when it cannot be reached that way (the caller then sends through the landing windows).  Opens the receiver's
// allocation on first use.
uint8_t* wire_map_mr(WirePair* p, uint32_t rkey, uint64_t addr, uint64_t bytes) {
  const uint32_t i = (rkey & 0xffu) - 1, gen = rkey >> 8;
  if (!g_par.wire_direct || rkey == 0 || i >= kPairMrs) return nullptr;
  std::lock_guard<std::mutex> g(p->mr_mu);
  auto& m = p->mr_map[i];
  if (!m.ptr || m.gen != gen) {
    DeviceScope keep;
    if (hipSetDevice(p->hip_device) != hipSuccess) return nullptr;
    if (m.ptr) { (void)hipIpcCloseMemHandle(m.ptr); m.ptr = nullptr; }
    const ShmMr& sm = p->w->mr[i];
    const uint32_t now = sm.gen.load(std::memory_order_acquire);
    if ((now & 0xffffffu) != gen || !(now & 1u) || sm.size >= (2ull << 30)) return nullptr;
    void* ptr = nullptr;
    if (hipIpcOpenMemHandle(&ptr, sm.handle, hipIpcMemLazyEnablePeerAccess) != hipSuccess) { (void)hipGetLastError(); return nullptr; }
    m.ptr = (uint8_t*)ptr;
    m.gen = gen;
    m.base = sm.base;
    m.size = sm.size;
  }
  if (addr < m.base || addr + bytes > m.base + m.size) return nullptr;
  return m.ptr + (addr - m.base);
}

// ---- sender ---------------------------------------------------------------------------------------------------------
// Is a set of landing windows free?  (launch_mu held: the only place waves are added.)
bool wire_set_free(WirePair* p) {
  uint64_t launched;
  {
    std::lock_guard<std::mutex> g(p->tx_mu);
    launched = p->tx_launched;
  }
  return launched - p->w->waves_consumed.load(std::memory_order_acquire) < (uint64_t)p->sets;
}
// the set the next wave lands in, and its number (launch_mu held)
uint32_t wire_next_set(WirePair* p, uint64_t* wave_no) {
  std::lock_guard<std::mutex> g(p->tx_mu);
  *wave_no = p->tx_launched + 1;
  return (uint32_t)(p->tx_launched % (uint64_t)p->sets);
}
// the wave's GPU work has been handed over (launch_mu held)
void wire_push_flight(WirePair* p, const WireFlight& f) {
  std::lock_guard<std::mutex> g(p->tx_mu);
  p->tx_flights.push_back(f);
  p->tx_launched++;
}

bool wire_flight_complete(Peer* pr, const WireFlight& f, ncclResult_t* rc);

// Announce the waves whose bytes have landed, in order: the stand-in for the WRITE_WITH_IMM completions
// (plugin.cc:1453-1465).  Any thread that polls a send of the pair comes through here; one at a time does the work.
ncclResult_t wire_publish(WirePair* p) {
  if (!p->tx_mu.try_lock()) return ncclSuccess;
  ncclResult_t rc = ncclSuccess;
  while (!p->tx_flights.empty()) {
    const WireFlight& f = p->tx_flights.front();
    if (!wire_flight_complete(p->peer, f, &rc)) break;
    if (rc != ncclSuccess) {   // the wave is lost: nothing behind it can be delivered in order
      p->w->failed.store(1, std::memory_order_release);
      break;
    }
    const uint64_t n = p->tx_published.load(std::memory_order_relaxed) + 1;
    ShmWave& wv = p->w->wave[(n - 1) % kPairWaves];
    memcpy((char*)&wv + sizeof(wv.seq), (const char*)&f.rec + sizeof(f.rec.seq), sizeof(ShmWave) - sizeof(wv.seq));
    wv.seq.store(n, std::memory_order_release);
    p->tx_published.store(n, std::memory_order_release);
    tl_event(7, n);
    p->tx_flights.pop_front();
  }
  p->tx_mu.unlock();
  return rc;
}

// ---- receiver -------------------------------------------------------------------------------------------------------
ncclResult_t wire_deliver(WirePair* p, const ShmWave& wv, WireFlight& f);

// Take the waves that have been announced off the ring and hand their delivery to the GPU; give the landing sets of
// delivered waves back, in order.  Any thread that polls a receive of the pair comes through here; one at a time works.
ncclResult_t wire_progress_recv(WirePair* p) {
  if (!p->rx_mu.try_lock()) return ncclSuccess;
  ncclResult_t rc = ncclSuccess;
  Peer* pr = p->peer;
  if (p->named && p->w->sender_mapped.load(std::memory_order_acquire)) {
    shm_unlink(p->name);   // both ends hold their mapping: the name is no longer needed and cannot leak
    p->named = false;
  }
  while (!p->rx_flights.empty()) {
    if (!wire_flight_complete(pr, p->rx_flights.front(), &rc)) break;
    // (a delivery that failed has failed its requests already; its set goes back all the same)
    rc = ncclSuccess;
    p->rx_done++;
    p->w->waves_consumed.store(p->rx_done, std::memory_order_release);
    p->rx_flights.pop_front();
  }
  for (;;) {
    const uint64_t taken = p->rx_taken.load(std::memory_order_relaxed);
    const ShmWave& wv = p->w->wave[taken % kPairWaves];
    if (wv.seq.load(std::memory_order_acquire) != taken + 1) break;         // nothing further has landed
    if (!pr->launch_mu.try_lock()) break;                                    // somebody is launching: next poll
    WireFlight f;
    tl_event(8, taken + 1);
    rc = wire_deliver(p, wv, f);
    pr->launch_mu.unlock();
    p->rx_taken.store(taken + 1, std::memory_order_release);
    p->rx_flights.push_back(f);
    if (rc != ncclSuccess) { p->w->failed.store(1, std::memory_order_release); break; }
  }
  p->rx_mu.unlock();
  return rc;
}
