// fl_plugin_shm_wire.h -- the plugin's wire between two processes.  Not a header of its own: fl_plugin.cc includes it
// inside its unnamed namespace, behind the objects and helpers it uses (Params, FifoWire, MemHandle, Handle, the request
// type codes, DeviceScope, FL_HIPCHECK / FL_FLHCHECK, ensure_pool, current_credits, wave_chunks) and in front of the
// entry points that dispatch to it by magic number.
// ------------------------------------------------------------------------------------------------
// shared-memory wire: sender and receiver in different processes (NCCL_FUSELINK_WIRE=shm)
// ------------------------------------------------------------------------------------------------
// The reference's two ends are different processes on different hosts: the receiver writes 64-byte descriptors into a
// FIFO in the sender's memory by RDMA (ncclIbSendFifo, plugin.cc:487-496, 1616-1677), the sender RDMA-writes the payload
// out of its staged buffer into the receiver's registered memory and completes it with a WRITE_WITH_IMM
// (plugin.cc:1453-1495), and the 128-byte handle that listen fills carries what connect needs to reach the listener
// (plugin.cc:425-430, 776-885).  On one GPU the part of that which can be shown is the process boundary: listen creates a
// POSIX shared-memory object and names it in the handle; connect, in another process, maps it.  The object holds the
// descriptor FIFO (receiver writes, sender reads), a ring of wave completions (sender writes, receiver reads: the
// stand-in for the WRITE_WITH_IMM completions) and the IPC handle of the receiver's landing windows.  A send then runs
// as in the reference's layers: the striping kernel stages a wave of the request's chunks in the sender's lane windows
// (HIP VMM, from the unit pool); the wire carries every lane's staged bytes into the receiver's landing window for that
// lane (one launch, flh_copy_runs), device memory of the receiver's process that the sender has opened through
// hipIpcOpenMemHandle (an imported VMM allocation would be the closer analogue; this runtime refuses
// hipMemImportFromShareableHandle for another process's descriptor, so the landing windows are a plain device
// allocation); the sender publishes the wave; the receiver's reassembly kernel writes the posted buffer from its landing
// windows and hands them back.  The receiver keeps NCCL_FUSELINK_WIRE_SETS sets of landing windows, so that many waves
// are on the wire at once; requests start, finish and are reported in order.
void fill_uniform(flh_uniform_params& u, const uint32_t* credits, uint64_t bytes, uint64_t src_base, uint64_t epoch_bytes, uint32_t tile);

constexpr uint64_t kHandleMagicShm = 0x4655534c53484d31ull;   // "FUSLSHM1"
constexpr uint32_t kShmCommMagic = 0x464c5343;                // "FLSC"
constexpr uint32_t kShmReqMagic = 0x464c5352;                 // "FLSR"
constexpr uint32_t kShmListenMagic = 0x464c534c;              // "FLSL"

constexpr int kShmSetsMax = 8;
struct ShmWave {                   // one wave of chunks that has landed in the receiver's windows
  std::atomic<uint64_t> seq;       // wave number + 1, written last
  uint64_t fifo_idx;               // the descriptor (request) it belongs to
  uint64_t epoch_bytes;            // the connection's credit-epoch prefix the wave was scheduled from
  uint64_t offset;                 // byte offset of the wave in the request
  uint64_t bytes;
  uint32_t last;                   // the request's last wave
  uint32_t set;                    // the set of landing windows it lies in
  // A wave may instead carry n_req >= 2 whole requests, fifo_idx and the ones behind it, staged as one message of
  // `bytes` from epoch_bytes on (flh_stripe_batch with one segment); req_bytes are the sends' sizes.
  uint32_t n_req;
  uint32_t pad;
  uint64_t req_bytes[FLH_BATCH_MAX];
};
struct ShmWire {
  uint64_t magic;
  uint32_t lanes;
  uint32_t channelId;
  std::atomic<uint32_t> connected, accepted, send_closed, recv_closed;
  std::atomic<uint32_t> landing_ready;
  uint32_t landing_sets;           // sets of landing windows = waves that may be on the wire at once
  uint64_t landing_bytes_per_lane;
  hipIpcMemHandle_t landing;       // sets x lanes x landing_bytes_per_lane of the receiver's device memory
  alignas(64) FifoWire fifo[FL_NET_MAX_REQUESTS];          // plugin.cc:487-496: written by the receiver, idx last
  alignas(64) ShmWave wave[FL_NET_MAX_REQUESTS];
  alignas(64) std::atomic<uint64_t> waves_consumed;        // receiver: waves reassembled so far, in order (their landing windows are free again)
};

struct ShmRequest {
  uint32_t magic = 0;
  int type = kReqUnused;
  struct ShmComm* comm = nullptr;
  uint64_t fifo_idx = 0;           // 1-based descriptor number
  uint64_t size = 0;
  uint32_t credits[FLH_MAX_LANES] = {};
  // sender
  const uint8_t* src = nullptr;
  uint64_t launched = 0;           // bytes whose waves have been queued on the GPU
  bool all_launched = false;       // (a request of no bytes still takes one wave)
  uint64_t last_wave = 0;          // number (from 1) of the request's last wave, once all_launched
  bool refresh = false;
  // receiver
  uint8_t* dst = nullptr;
  uint64_t received = 0;           // bytes reassembled
  bool complete = false;           // the last wave has been reassembled
};

struct ShmFlight {                 // a wave whose GPU work is queued: the event of its set tells when it is through
  ShmRequest* req;
  uint64_t fifo_idx, epoch_bytes, offset, bytes;
  uint32_t last, set;
  uint32_t n_req = 1;              // a wave of several whole requests: req and the ones behind it
  ShmRequest* batch[FLH_BATCH_MAX];
  uint64_t req_bytes[FLH_BATCH_MAX];
};

struct ShmComm {
  uint32_t magic = kShmCommMagic;
  int is_send = 0;
  int dev = 0;
  ShmWire* w = nullptr;
  char name[64] = "";
  bool owner = false;              // the receiver created the object and unlinks it
  std::mutex mu;
  ShmRequest reqs[FL_NET_MAX_REQUESTS];
  uint64_t fifoHead = 0, fifoTail = 0;       // sender: next descriptor to match; receiver: next to post
  std::deque<ShmRequest*> active;            // requests in flight, in order: they start, finish and are reported in that order
  size_t cursor = 0;                         // sender: first request of `active` with waves left to launch; receiver: the one the next wave belongs to
  std::deque<ShmFlight> flights;             // waves queued on the GPU, in order
  uint64_t epoch_bytes = 0;                  // sender: the scheduler's carried prefix
  uint64_t waves_launched = 0;               // sender: waves queued on the GPU so far; receiver: waves taken off the wire so far
  uint64_t waves_published = 0;              // sender: waves announced to the receiver
  uint64_t waves_done = 0;                   // receiver: waves reassembled (what waves_consumed says)
  uint32_t last_rows = 0;                    // sender: chunks of the latest wave (rows of d_table)
  int64_t r_finished = 0, r_inflight = 0;
  int fuselink_offset = -1;
  uint8_t credits[FL_NET_MAX_LANES] = {};
  bool have_decision = false;
  // GPU side
  bool gpu_ready = false;
  int hip_device = -1;
  int sets = 0;
  hipStream_t stream = nullptr;
  hipEvent_t ev[kShmSetsMax] = {};           // one per set of landing windows: the latest wave that uses the set
  flh_window* win[FL_NET_MAX_LANES] = {};    // sender: staging windows
  flh_windows wins = {};
  uint8_t* landing = nullptr;                // receiver: its allocation; sender: the same memory opened through IPC
  flh_windows landing_wins[kShmSetsMax] = {};
  flh_chunk_desc* d_table = nullptr;
  flh_sched_hdr* d_hdr = nullptr;
  int32_t *h_status = nullptr, *d_status = nullptr;
};

struct ShmListen {
  uint32_t magic = kShmListenMagic;
  int dev = 0;
  ShmComm* comm = nullptr;         // becomes the recv comm at accept
};

std::atomic<uint64_t> g_shm_counter{0};

void shm_comm_free(ShmComm* c) {
  if (c->stream) {
    DeviceScope keep;
    (void)hipSetDevice(c->hip_device);
    (void)hipStreamSynchronize(c->stream);
    for (int l = 0; l < FL_NET_MAX_LANES; ++l) if (c->win[l]) (void)flh_window_destroy(c->win[l]);
    if (c->landing) { if (c->is_send) (void)hipIpcCloseMemHandle(c->landing); else (void)hipFree(c->landing); }
    if (c->d_table) (void)hipFree(c->d_table);
    if (c->d_hdr) (void)hipFree(c->d_hdr);
    if (c->h_status) (void)hipHostFree(c->h_status);
    for (hipEvent_t e : c->ev) if (e) (void)hipEventDestroy(e);
    (void)hipStreamDestroy(c->stream);
  }
  if (c->w) munmap(c->w, sizeof(ShmWire));
  if (c->owner && c->name[0]) shm_unlink(c->name);
  delete c;
  g_live_links.fetch_sub(1);   // (a reset of the plugin waits for these as for the in-process connections)
}

ncclResult_t shm_listen(int dev, void* opaqueHandle, void** listenComm) {
  ShmListen* lc = new (std::nothrow) ShmListen();
  ShmComm* c = new (std::nothrow) ShmComm();
  if (!lc || !c) { delete lc; delete c; return ncclSystemError; }
  g_live_links.fetch_add(1);
  snprintf(c->name, sizeof(c->name), "/fuselink-wire-%d-%llu", (int)getpid(), (unsigned long long)g_shm_counter.fetch_add(1));
  int fd = shm_open(c->name, O_CREAT | O_EXCL | O_RDWR, 0600);
  if (fd < 0 || ftruncate(fd, sizeof(ShmWire)) != 0) { if (fd >= 0) close(fd); FL_WARN("NET/FuseLink : shm_open(%s) failed", c->name); delete lc; delete c; g_live_links.fetch_sub(1); return ncclSystemError; }
  void* p = mmap(nullptr, sizeof(ShmWire), PROT_READ | PROT_WRITE, MAP_SHARED, fd, 0);
  close(fd);
  if (p == MAP_FAILED) { shm_unlink(c->name); delete lc; delete c; g_live_links.fetch_sub(1); return ncclSystemError; }
  memset(p, 0, sizeof(ShmWire));
  c->w = (ShmWire*)p;
  c->owner = true;
  c->dev = dev;
  c->w->lanes = (uint32_t)g_par.lanes;
  {
    std::lock_guard<std::mutex> g(g_reg_mu);
    c->w->channelId = (uint32_t)g_channel_counter++;
  }
  c->w->magic = kHandleMagicShm;
  lc->dev = dev;
  lc->comm = c;
  Handle* h = (Handle*)opaqueHandle;
  memset(h, 0, NCCL_NET_HANDLE_MAXSIZE);
  h->magic = kHandleMagicShm;
  h->channelId = (int32_t)c->w->channelId;
  h->dev = dev;
  // the object's name travels in the handle, as the listener's address does in the reference's (plugin.cc:425-430)
  static_assert(sizeof(Handle) + 64 <= NCCL_NET_HANDLE_MAXSIZE, "the name must fit behind the fixed part of the handle");
  memcpy((char*)opaqueHandle + sizeof(Handle), c->name, sizeof(c->name));
  *listenComm = lc;
  return ncclSuccess;
}

ncclResult_t shm_connect(int dev, void* opaqueHandle, void** sendComm) {
  Handle* h = (Handle*)opaqueHandle;
  *sendComm = nullptr;
  ShmComm* c = (ShmComm*)h->stage_link;
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
    c = new (std::nothrow) ShmComm();
    if (!c) { munmap(p, sizeof(ShmWire)); return ncclSystemError; }
    g_live_links.fetch_add(1);
    c->w = (ShmWire*)p;
    if (c->w->magic != kHandleMagicShm || (int)c->w->lanes != g_par.lanes) {
      FL_WARN("NET/FuseLink : connect: the listener runs %u lanes, this side %d", c->w->lanes, g_par.lanes);
      shm_comm_free(c);
      return ncclInvalidUsage;
    }
    int listener_pid = -1;
    if (sscanf(name, "/fuselink-wire-%d-", &listener_pid) == 1 && listener_pid == (int)getpid()) {
      // the landing windows reach the sender through HIP IPC, which a process cannot open on its own allocations
      FL_WARN("NET/FuseLink : NCCL_FUSELINK_WIRE=shm connects two processes; this listener lives in the connecting process (unset it for the in-process wire)");
      shm_comm_free(c);
      return ncclInvalidUsage;
    }
    c->is_send = 1;
    c->dev = dev;
    memcpy(c->name, name, sizeof(name));
    c->w->connected.store(1, std::memory_order_release);
    h->stage = 1;
    h->stage_link = c;
    return ncclSuccess;
  }
  if (!c->w->accepted.load(std::memory_order_acquire)) return ncclSuccess;   // accept has not happened yet
  h->stage = 0;
  h->stage_link = nullptr;
  *sendComm = c;
  return ncclSuccess;
}

ncclResult_t shm_accept(ShmListen* lc, void** recvComm) {
  *recvComm = nullptr;
  ShmComm* c = lc->comm;
  if (!c || !c->w->connected.load(std::memory_order_acquire)) return ncclSuccess;   // nobody connected yet
  c->w->accepted.store(1, std::memory_order_release);
  shm_unlink(c->name);   // both ends hold their mapping: the name is no longer needed and cannot leak
  c->owner = false;
  lc->comm = nullptr;
  *recvComm = c;
  return ncclSuccess;
}

// set k, lane l of the landing windows: one allocation, set after set, lane after lane
void shm_landing_windows(ShmComm* c, uint64_t per_lane) {
  for (int k = 0; k < c->sets; ++k) {
    c->landing_wins[k].n_lanes = (uint32_t)g_par.lanes;
    for (int l = 0; l < g_par.lanes; ++l) {
      c->landing_wins[k].base[l] = c->landing + ((uint64_t)k * (uint64_t)g_par.lanes + (uint64_t)l) * per_lane;
      c->landing_wins[k].cap[l] = per_lane;
    }
  }
}

// stream, status word, table buffers; the sender's staging windows or the receiver's landing windows
ncclResult_t shm_setup_gpu(ShmComm* c, int device) {
  if (c->gpu_ready) return ncclSuccess;
  if (c->stream) return ncclInternalError;   // failed earlier
  DeviceScope keep;
  c->hip_device = device;
  FL_HIPCHECK(hipSetDevice(device));
  FL_HIPCHECK(hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking));
  FL_HIPCHECK(hipHostMalloc((void**)&c->h_status, 64, hipHostMallocMapped));
  memset(c->h_status, 0, 64);
  FL_HIPCHECK(hipHostGetDevicePointer((void**)&c->d_status, c->h_status, 0));
  const uint64_t cap = (uint64_t)g_par.window_units * FLH_UNIT_BYTES;
  if (c->is_send) {
    flh_pool* pool = nullptr;
    ncclResult_t rc = ensure_pool(device, &pool);
    if (rc != ncclSuccess) return rc;
    c->wins.n_lanes = (uint32_t)g_par.lanes;
    for (int l = 0; l < g_par.lanes; ++l) {
      FL_FLHCHECK(flh_window_create(pool, cap, &c->win[l]));
      FL_FLHCHECK(flh_window_bind(c->win[l], cap));
      c->wins.base[l] = flh_window_base(c->win[l]);
      c->wins.cap[l] = flh_window_bound_bytes(c->win[l]);
    }
    FL_HIPCHECK(hipMalloc((void**)&c->d_table, sizeof(flh_chunk_desc) * (size_t)g_par.max_wave_chunks));
    FL_HIPCHECK(hipMalloc((void**)&c->d_hdr, sizeof(flh_sched_hdr)));
    // (the landing windows, and with them the number of sets and their events, come with the receiver's first descriptor)
  } else {
    c->sets = g_par.wire_sets;
    const uint64_t bytes = cap * (uint64_t)g_par.lanes * (uint64_t)c->sets;
    if (bytes >= (2ull << 30)) { FL_WARN("NET/FuseLink : %d sets of landing windows take %llu bytes; a shared allocation must stay under 2 GiB", c->sets, (unsigned long long)bytes); return ncclInvalidUsage; }
    FL_HIPCHECK(hipMalloc((void**)&c->landing, bytes));
    FL_HIPCHECK(hipIpcGetMemHandle(&c->w->landing, c->landing));
    c->w->landing_bytes_per_lane = cap;
    c->w->landing_sets = (uint32_t)c->sets;
    for (int k = 0; k < c->sets; ++k) FL_HIPCHECK(hipEventCreateWithFlags(&c->ev[k], hipEventDisableTiming));
    shm_landing_windows(c, cap);
    c->w->landing_ready.store(1, std::memory_order_release);
  }
  c->gpu_ready = true;
  return ncclSuccess;
}

ShmRequest* shm_get_request(ShmComm* c, int type) {
  for (int i = 0; i < FL_NET_MAX_REQUESTS; ++i) {
    ShmRequest* r = &c->reqs[i];
    if (r->type == kReqUnused) {
      *r = ShmRequest();
      r->magic = kShmReqMagic;
      r->type = type;
      r->comm = c;
      return r;
    }
  }
  FL_WARN("NET/FuseLink : unable to allocate requests");
  return nullptr;
}

// Credit row a descriptor asks for (both ends derive it from the descriptor alone, so they agree).
void shm_wire_credits(const ShmComm* c, const FifoWire& w, uint32_t* credits) {
  for (int l = 0; l < FLH_MAX_LANES; ++l) credits[l] = 0;
  if (w.fuselink_offset == -2) { for (int l = 0; l < g_par.lanes; ++l) credits[l] = w.credits[l]; }
  else credits[w.fuselink_offset >= 0 ? w.fuselink_offset % g_par.lanes : (int)(c->w->channelId % (uint32_t)g_par.lanes)] = 1;
}

ncclResult_t shm_irecv(ShmComm* c, void* data, int size, int tag, MemHandle* mh, void** request) {
  *request = nullptr;
  if (mh->type != NCCL_PTR_CUDA) { FL_WARN("NET/FuseLink : the shared-memory wire carries device memory only"); return ncclInvalidUsage; }
  std::lock_guard<std::mutex> g(c->mu);
  ncclResult_t rc = shm_setup_gpu(c, mh->device);
  if (rc != ncclSuccess) return rc;
  bool refreshed = false;
  if (c->r_finished % g_par.refresh_batch == 0 || !c->have_decision) {   // plugin.cc:1700-1712
    if (c->r_inflight != 0) return ncclSuccess;
    if (g_par.policy == 0) {
      c->fuselink_offset = (int)(c->w->channelId % (uint32_t)g_par.lanes);
    } else {
      c->fuselink_offset = -2;
      current_credits(c->dev % g_par.lanes, c->credits);
    }
    c->have_decision = true;
    refreshed = true;
  }
  if ((int)c->active.size() >= FL_NET_MAX_REQUESTS - 1) return ncclSuccess;   // the descriptor ring is full
  ShmRequest* r = shm_get_request(c, kReqRecv);
  if (!r) return ncclInternalError;
  r->dst = (uint8_t*)data;
  r->size = (uint64_t)size;
  r->fifo_idx = c->fifoTail + 1;
  FifoWire& w = c->w->fifo[c->fifoTail % FL_NET_MAX_REQUESTS];
  w.addr = (uint64_t)(uintptr_t)data;
  w.size = size;
  w.rkey = 1;
  w.nreqs = 1;
  w.tag = (uint32_t)tag;
  w.fuselink_offset = c->fuselink_offset;
  memcpy(w.credits, c->credits, sizeof(w.credits));
  w.flags = refreshed ? 1u : 0u;
  shm_wire_credits(c, w, r->credits);
  __atomic_store_n(&w.idx, c->fifoTail + 1, __ATOMIC_RELEASE);   // written last: it is what the sender waits for (plugin.cc:1632)
  c->fifoTail++;
  c->r_inflight++;
  c->active.push_back(r);
  *request = r;
  return ncclSuccess;
}

ncclResult_t shm_isend(ShmComm* c, void* data, int size, int tag, MemHandle* mh, void** request) {
  *request = nullptr;
  if (mh->type != NCCL_PTR_CUDA) { FL_WARN("NET/FuseLink : the shared-memory wire carries device memory only"); return ncclInvalidUsage; }
  std::lock_guard<std::mutex> g(c->mu);
  FifoWire& fw = c->w->fifo[c->fifoHead % FL_NET_MAX_REQUESTS];
  if (__atomic_load_n(&fw.idx, __ATOMIC_ACQUIRE) != c->fifoHead + 1) return ncclSuccess;   // not posted yet (plugin.cc:1510-1514)
  if (fw.nreqs != 1) return ncclInternalError;
  if (fw.tag != (uint32_t)tag) return ncclSuccess;
  if (size > fw.size) { FL_WARN("NET/FuseLink : req tag %x collective mismatch error, local size %d remote size %d", tag, size, fw.size); return ncclInvalidUsage; }
  ncclResult_t rc = shm_setup_gpu(c, mh->device);
  if (rc != ncclSuccess) return rc;
  if (!c->landing) {   // the receiver's landing windows, once it has set them up
    if (!c->w->landing_ready.load(std::memory_order_acquire)) return ncclSuccess;
    DeviceScope keep;
    FL_HIPCHECK(hipSetDevice(c->hip_device));
    if (c->w->landing_bytes_per_lane < c->wins.cap[0] || c->w->landing_sets < 1 || c->w->landing_sets > (uint32_t)kShmSetsMax) {
      FL_WARN("NET/FuseLink : the receiver's landing windows (%u sets of %llu bytes per lane) do not fit this side's staging windows",
              c->w->landing_sets, (unsigned long long)c->w->landing_bytes_per_lane);
      return ncclInvalidUsage;
    }
    FL_HIPCHECK(hipIpcOpenMemHandle((void**)&c->landing, c->w->landing, hipIpcMemLazyEnablePeerAccess));
    c->sets = (int)c->w->landing_sets;
    for (int k = 0; k < c->sets; ++k) FL_HIPCHECK(hipEventCreateWithFlags(&c->ev[k], hipEventDisableTiming));
    shm_landing_windows(c, c->w->landing_bytes_per_lane);
  }
  ShmRequest* r = shm_get_request(c, kReqSend);
  if (!r) return ncclInternalError;
  r->src = (const uint8_t*)data;
  r->size = (uint64_t)size;
  r->fifo_idx = c->fifoHead + 1;
  r->refresh = (fw.flags & 1u) != 0;
  shm_wire_credits(c, fw, r->credits);
  memset((void*)&fw, 0, sizeof(FifoWire));   // plugin.cc:1605
  c->fifoHead++;
  c->active.push_back(r);
  *request = r;
  return ncclSuccess;
}

// The sender's side of the wire (c->mu held): queue waves on the GPU while sets of landing windows are free, announce
// the waves whose copies have finished.  A wave is the striping launch into this side's staging windows plus one launch
// that carries every lane's staged bytes into the receiver's landing windows of the wave's set; launches of one stream
// run in order, so the next wave's striping cannot overtake the copy that still reads the staging windows.
ncclResult_t shm_progress_send(ShmComm* c) {
  const uint64_t chunk = (uint64_t)g_par.chunk;
  DeviceScope keep;
  bool device_set = false;
  // announce what has landed: the stand-in for the WRITE_WITH_IMM completions (plugin.cc:1453-1465)
  while (!c->flights.empty()) {
    const ShmFlight& f = c->flights.front();
    hipError_t e = hipEventQuery(c->ev[f.set]);
    if (e == hipErrorNotReady) break;
    if (e != hipSuccess) return hip_fail("hipEventQuery", e);
    if (*(volatile int32_t*)c->h_status != 0) { FL_WARN("NET/FuseLink : a chunk fell outside its staging window (status %d)", *c->h_status); return ncclInternalError; }
    ShmWave& wv = c->w->wave[c->waves_published % FL_NET_MAX_REQUESTS];
    wv.fifo_idx = f.fifo_idx;
    wv.epoch_bytes = f.epoch_bytes;
    wv.offset = f.offset;
    wv.bytes = f.bytes;
    wv.last = f.last;
    wv.set = f.set;
    wv.n_req = f.n_req;
    for (uint32_t q = 0; q < f.n_req && f.n_req > 1; ++q) wv.req_bytes[q] = f.req_bytes[q];
    c->waves_published++;
    wv.seq.store(c->waves_published, std::memory_order_release);
    c->flights.pop_front();
  }
  // queue further waves: a set of landing windows is free once the wave that used it last has been reassembled
  while (c->cursor < c->active.size()) {
    ShmRequest* r = c->active[c->cursor];
    if (r->all_launched) { c->cursor++; continue; }
    const uint64_t consumed = c->w->waves_consumed.load(std::memory_order_acquire);
    if (c->waves_launched - consumed >= (uint64_t)c->sets) {
      if (c->w->recv_closed.load(std::memory_order_acquire)) { FL_WARN("NET/FuseLink : the receiving process closed the connection with a wave outstanding"); return ncclRemoteError; }
      break;
    }
    if (r->refresh && r->launched == 0) c->epoch_bytes = 0;
    uint64_t wave = (uint64_t)wave_chunks(r->credits, g_par.lanes, chunk, c->wins.cap[0], c->epoch_bytes / chunk) * chunk;
    const uint64_t room = wave;
    if (wave > r->size - r->launched) wave = r->size - r->launched;
    const uint32_t set = (uint32_t)(c->waves_launched % (uint64_t)c->sets);
    if (!device_set) { FL_HIPCHECK(hipSetDevice(c->hip_device)); device_set = true; }
    // Requests behind this one that have not started either, under the same credit row and without a refresh of
    // their own, share the wave while it has room: together they are one message from the carried prefix on (every
    // request but the last a whole number of chunks), staged by one launch, carried by one, reassembled by one.  At
    // NCCL's 512 KiB steps a wave per request costs both sides their launches and events for half a megabyte each.
    uint32_t n_req = 1;
    uint64_t total = r->size;
    if (g_par.wire_batch > 1 && r->launched == 0 && r->size > 0 && r->size <= room) {
      while ((int)n_req < g_par.wire_batch && c->cursor + n_req < c->active.size()) {
        const ShmRequest* prev = c->active[c->cursor + n_req - 1];
        const ShmRequest* t = c->active[c->cursor + n_req];
        if (prev->size % chunk != 0 || t->refresh || t->size == 0 || t->launched != 0 || t->all_launched ||
            memcmp(t->credits, r->credits, sizeof(r->credits)) != 0 || total + t->size > room)
          break;
        total += t->size;
        ++n_req;
      }
    }
    if (n_req >= 2) {
      flh_batch_params b;
      memset(&b, 0, sizeof(b));
      fill_uniform(b.u, r->credits, total, 0, c->epoch_bytes, FLH_TILE_BYTES);
      b.n_req = n_req;
      ShmFlight f;
      for (uint32_t q = 0; q < n_req; ++q) {
        ShmRequest* t = c->active[c->cursor + q];
        b.d_src[q] = t->src;
        b.bytes[q] = t->size;
        f.batch[q] = t;
        f.req_bytes[q] = t->size;
      }
      FL_FLHCHECK(flh_stripe_batch(&b, &c->wins, c->d_table, c->d_hdr, c->d_status, c->stream));
      c->last_rows = (uint32_t)((total + chunk - 1) / chunk);
      FlCreditRow row;
      fl_row_make(r->credits, (uint32_t)g_par.lanes, row);
      uint64_t lane_bytes[FLH_MAX_LANES];
      uint32_t lane_chunks[FLH_MAX_LANES];
      fl_row_lane_totals(row, c->epoch_bytes / chunk, total, chunk, lane_bytes, lane_chunks);
      FL_FLHCHECK(flh_copy_runs(c->landing_wins[set].base, c->wins.base, lane_bytes, (uint32_t)g_par.lanes, c->stream));
      FL_HIPCHECK(hipEventRecord(c->ev[set], c->stream));
      f.req = r;
      f.fifo_idx = r->fifo_idx;
      f.epoch_bytes = c->epoch_bytes;
      f.offset = 0;
      f.bytes = total;
      f.set = set;
      f.last = 1;
      f.n_req = n_req;
      c->epoch_bytes += total;
      c->waves_launched++;
      for (uint32_t q = 0; q < n_req; ++q) {
        ShmRequest* t = f.batch[q];
        t->launched = t->size;
        t->all_launched = true;
        t->last_wave = c->waves_launched;
      }
      c->flights.push_back(f);
      continue;   // the cursor steps over the requests at the top of the loop
    }
    if (wave) {
      flh_uniform_params u;
      fill_uniform(u, r->credits, wave, r->launched, c->epoch_bytes, FLH_TILE_BYTES);
      FL_FLHCHECK(flh_stripe_uniform(r->src, r->size, &c->wins, &u, c->d_table, c->d_hdr, c->d_status, c->stream));
      c->last_rows = (uint32_t)((wave + chunk - 1) / chunk);
      // the wire: every lane's staged bytes into the receiver's landing window of that lane, one launch for all lanes
      FlCreditRow row;
      fl_row_make(r->credits, (uint32_t)g_par.lanes, row);
      uint64_t lane_bytes[FLH_MAX_LANES];
      uint32_t lane_chunks[FLH_MAX_LANES];
      fl_row_lane_totals(row, c->epoch_bytes / chunk, wave, chunk, lane_bytes, lane_chunks);
      FL_FLHCHECK(flh_copy_runs(c->landing_wins[set].base, c->wins.base, lane_bytes, (uint32_t)g_par.lanes, c->stream));
    }
    FL_HIPCHECK(hipEventRecord(c->ev[set], c->stream));
    ShmFlight f;
    f.req = r;
    f.fifo_idx = r->fifo_idx;
    f.epoch_bytes = c->epoch_bytes;
    f.offset = r->launched;
    f.bytes = wave;
    f.set = set;
    c->epoch_bytes += wave;
    r->launched += wave;
    c->waves_launched++;
    f.last = r->launched >= r->size ? 1u : 0u;
    if (f.last) { r->all_launched = true; r->last_wave = c->waves_launched; }
    c->flights.push_back(f);
  }
  return ncclSuccess;
}

// The receiver's side (c->mu held): reassemble the waves that have been announced out of their landing windows, and
// hand the windows back, in order, as the reassembly launches finish.
ncclResult_t shm_progress_recv(ShmComm* c) {
  DeviceScope keep;
  bool device_set = false;
  while (!c->flights.empty()) {
    const ShmFlight& f = c->flights.front();
    hipError_t e = hipEventQuery(c->ev[f.set]);
    if (e == hipErrorNotReady) break;
    if (e != hipSuccess) return hip_fail("hipEventQuery", e);
    if (*(volatile int32_t*)c->h_status != 0) { FL_WARN("NET/FuseLink : a chunk fell outside its landing window or buffer (status %d)", *c->h_status); return ncclInternalError; }
    if (f.n_req > 1) {
      for (uint32_t q = 0; q < f.n_req; ++q) { f.batch[q]->received += f.req_bytes[q]; f.batch[q]->complete = true; }
    } else {
      f.req->received += f.bytes;
      if (f.last) f.req->complete = true;
    }
    c->waves_done++;
    c->w->waves_consumed.store(c->waves_done, std::memory_order_release);   // the set's landing windows are free again
    c->flights.pop_front();
  }
  for (;;) {
    ShmWave& wv = c->w->wave[c->waves_launched % FL_NET_MAX_REQUESTS];
    if (wv.seq.load(std::memory_order_acquire) != c->waves_launched + 1) {   // nothing further has landed
      if (c->cursor < c->active.size() && c->w->send_closed.load(std::memory_order_acquire)) {
        FL_WARN("NET/FuseLink : the sending process closed the connection with a receive outstanding");
        return ncclRemoteError;
      }
      break;
    }
    if (c->cursor >= c->active.size()) { FL_WARN("NET/FuseLink : a wave arrived that no posted receive is waiting for"); return ncclInternalError; }
    ShmRequest* r = c->active[c->cursor];
    if (wv.fifo_idx != r->fifo_idx) {
      FL_WARN("NET/FuseLink : a wave of request %llu arrived while %llu is next in line", (unsigned long long)wv.fifo_idx, (unsigned long long)r->fifo_idx);
      return ncclInternalError;
    }
    if (wv.set >= (uint32_t)c->sets) { FL_WARN("NET/FuseLink : a wave in a set of landing windows that does not exist"); return ncclInvalidUsage; }
    if (wv.n_req > 1) {
      // several whole requests in one wave: this receive and the ones posted behind it
      const uint32_t n_req = wv.n_req;
      if (n_req > FLH_BATCH_MAX || c->cursor + n_req > c->active.size()) { FL_WARN("NET/FuseLink : a wave of %u requests arrived, %zu receives are posted", n_req, c->active.size() - c->cursor); return ncclInternalError; }
      if (!device_set) { FL_HIPCHECK(hipSetDevice(c->hip_device)); device_set = true; }
      flh_batch_params b;
      memset(&b, 0, sizeof(b));
      fill_uniform(b.u, r->credits, wv.bytes, 0, wv.epoch_bytes, FLH_TILE_BYTES);
      b.n_req = n_req;
      ShmFlight f;
      uint64_t sum = 0;
      for (uint32_t q = 0; q < n_req; ++q) {
        ShmRequest* t = c->active[c->cursor + q];
        if (t->fifo_idx != wv.fifo_idx + q || wv.req_bytes[q] > t->size || memcmp(t->credits, r->credits, sizeof(r->credits)) != 0) {
          FL_WARN("NET/FuseLink : request %u of a wave does not fit the receive posted for it", q);
          return ncclInvalidUsage;
        }
        b.d_dst[q] = t->dst;
        b.bytes[q] = wv.req_bytes[q];
        f.batch[q] = t;
        f.req_bytes[q] = wv.req_bytes[q];
        sum += wv.req_bytes[q];
      }
      if (sum != wv.bytes) { FL_WARN("NET/FuseLink : a wave's requests do not add up to its bytes"); return ncclInvalidUsage; }
      FL_FLHCHECK(flh_reassemble_batch(&b, &c->landing_wins[wv.set], c->d_status, c->stream));
      FL_HIPCHECK(hipEventRecord(c->ev[wv.set], c->stream));
      f.req = r;
      f.fifo_idx = wv.fifo_idx;
      f.epoch_bytes = wv.epoch_bytes;
      f.offset = 0;
      f.bytes = wv.bytes;
      f.last = 1;
      f.set = wv.set;
      f.n_req = n_req;
      c->flights.push_back(f);
      c->waves_launched++;
      c->cursor += n_req;
      continue;
    }
    if (wv.offset + wv.bytes > r->size) { FL_WARN("NET/FuseLink : a wave past the end of the posted buffer"); return ncclInvalidUsage; }
    if (!device_set) { FL_HIPCHECK(hipSetDevice(c->hip_device)); device_set = true; }
    if (wv.bytes) {
      // the credit row this receiver put into the descriptor: the reassembly launch derives the same lanes and offsets
      flh_uniform_params u;
      fill_uniform(u, r->credits, wv.bytes, wv.offset, wv.epoch_bytes, FLH_TILE_BYTES);
      FL_FLHCHECK(flh_reassemble_uniform(r->dst, r->size, &c->landing_wins[wv.set], &u, c->d_status, c->stream));
    }
    FL_HIPCHECK(hipEventRecord(c->ev[wv.set], c->stream));
    ShmFlight f;
    f.req = r;
    f.fifo_idx = wv.fifo_idx;
    f.epoch_bytes = wv.epoch_bytes;
    f.offset = wv.offset;
    f.bytes = wv.bytes;
    f.last = wv.last;
    f.set = wv.set;
    c->flights.push_back(f);
    c->waves_launched++;
    if (wv.last) c->cursor++;   // the next wave belongs to the next receive
  }
  return ncclSuccess;
}

// The table and header that the striping launch of the connection's latest wave wrote (control surface, for tests).
int shm_last_table(ShmComm* c, void* rows_out, int max_rows, void* hdr_out) {
  std::lock_guard<std::mutex> g(c->mu);
  if (!c->gpu_ready || c->last_rows == 0) return fl_set_error(FLH_E_STATE, "the connection has not staged anything yet");
  DeviceScope keep;
  if (hipSetDevice(c->hip_device) != hipSuccess) return fl_set_error(FLH_E_HIP, "hipSetDevice failed");
  if (hipStreamSynchronize(c->stream) != hipSuccess) return fl_set_error(FLH_E_HIP, "stream synchronize failed");
  const int rows = (int)c->last_rows, take = rows < max_rows ? rows : max_rows;
  if (take > 0 && rows_out && hipMemcpy(rows_out, c->d_table, sizeof(flh_chunk_desc) * (size_t)take, hipMemcpyDeviceToHost) != hipSuccess)
    return fl_set_error(FLH_E_HIP, "table copy failed");
  if (hdr_out && hipMemcpy(hdr_out, c->d_hdr, sizeof(flh_sched_hdr), hipMemcpyDeviceToHost) != hipSuccess)
    return fl_set_error(FLH_E_HIP, "header copy failed");
  return rows;
}

ncclResult_t shm_test(ShmRequest* r, int* done, int* sizes) {
  *done = 0;
  ShmComm* c = r->comm;
  std::lock_guard<std::mutex> g(c->mu);
  ncclResult_t rc = c->is_send ? shm_progress_send(c) : shm_progress_recv(c);
  if (rc != ncclSuccess) return rc;
  if (c->active.empty() || c->active.front() != r) return ncclSuccess;   // requests are reported in the order they were made
  if (r->type == kReqSend) {
    // the send is complete once its last wave has been taken out of the landing windows
    if (!r->all_launched || c->w->waves_consumed.load(std::memory_order_acquire) < r->last_wave) {
      if (r->all_launched && c->w->recv_closed.load(std::memory_order_acquire)) {
        FL_WARN("NET/FuseLink : the receiving process closed the connection with a wave outstanding");
        return ncclRemoteError;
      }
      return ncclSuccess;
    }
  } else {
    if (!r->complete) return ncclSuccess;
    c->r_finished++;
    c->r_inflight--;
    if (sizes) sizes[0] = (int)r->received;
  }
  c->active.pop_front();
  if (c->cursor) c->cursor--;
  r->type = kReqUnused;
  *done = 1;
  return ncclSuccess;
}

