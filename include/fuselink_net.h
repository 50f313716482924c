/*
 * fuselink_net.h -- the NCCL/RCCL network-plugin ABI exported by libnccl-net-fuselink.so.
 *
 * Self-contained restatement of the ext-net structures (no nccl.h needed).  The reference exports
 * `ncclNetPlugin_v7` and aliases `ncclNetPlugin_v6` to it (FuseLink src/plugin.cc:1997-2018; struct
 * definitions in src/extern/nccl_net.h:24-98 for v7 and :104-163 for v6).  This library exports
 *     ncclNetPlugin_v8   (primary: what RCCL 2.2x probes first among the versions carried here)
 *     ncclNetPlugin_v7   (the reference's own version)
 *     ncclNetPlugin_v6   (a real v6 table; the reference's alias relies on the v7 and v6 layouts
 *                         agreeing in their leading slots)
 * v8 differs from v7 in two places only: regMr takes `size_t size` instead of `int size`, and the
 * properties struct gains `int regIsGlobal` after ptrSupport.
 *
 * Calling convention (src/extern/nccl_net.h:53-83): every entry returns ncclResult_t; "would block"
 * is ncclSuccess with *sendComm / *recvComm / *request left NULL and the call is repeated.
 */
#ifndef FUSELINK_NET_H_
#define FUSELINK_NET_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- result codes (values of rccl.h / nccl.h) ---------------------------------------------- */
#ifndef NCCL_H_
typedef enum {
  ncclSuccess = 0,
  ncclUnhandledCudaError = 1,
  ncclSystemError = 2,
  ncclInternalError = 3,
  ncclInvalidArgument = 4,
  ncclInvalidUsage = 5,
  ncclRemoteError = 6,
  ncclInProgress = 7,
  ncclNumResults = 8
} ncclResult_t;
#endif

/* ---- logging (nccl_common.h of NCCL 2.19) -------------------------------------------------- */
typedef enum { NCCL_LOG_NONE = 0, NCCL_LOG_VERSION = 1, NCCL_LOG_WARN = 2, NCCL_LOG_INFO = 3, NCCL_LOG_ABORT = 4, NCCL_LOG_TRACE = 5 } ncclDebugLogLevel;
typedef enum {
  NCCL_INIT = 1, NCCL_COLL = 2, NCCL_P2P = 4, NCCL_SHM = 8, NCCL_NET = 16, NCCL_GRAPH = 32, NCCL_TUNING = 64,
  NCCL_ENV = 128, NCCL_ALLOC = 256, NCCL_CALL = 512, NCCL_PROXY = 1024, NCCL_NVLS = 2048, NCCL_ALL = ~0
} ncclDebugLogSubSys;
typedef void (*ncclDebugLogger_t)(ncclDebugLogLevel level, unsigned long flags, const char* file, int line, const char* fmt, ...);

/* ---- constants (src/extern/nccl_net.h:15-22) ----------------------------------------------- */
#define NCCL_NET_HANDLE_MAXSIZE 128
#define NCCL_PTR_HOST 0x1
#define NCCL_PTR_CUDA 0x2
#define NCCL_PTR_DMABUF 0x4
#define NCCL_NET_MAX_REQUESTS 32

/* ---- device offload descriptors (net_device.h) ---------------------------------------------- */
typedef enum { NCCL_NET_DEVICE_HOST = 0, NCCL_NET_DEVICE_UNPACK = 1 } ncclNetDeviceType;
#define NCCL_NET_DEVICE_INVALID_VERSION 0x0
typedef struct {
  ncclNetDeviceType netDeviceType;
  int netDeviceVersion;
  void* handle;
  size_t size;
  int needsProxyProgress;
} ncclNetDeviceHandle_v7_t;
typedef ncclNetDeviceHandle_v7_t ncclNetDeviceHandle_v8_t;

/* ---- properties ------------------------------------------------------------------------------- */
typedef struct {  /* src/extern/nccl_net.h:105-116 */
  char* name;
  char* pciPath;
  uint64_t guid;
  int ptrSupport;
  int speed;
  int port;
  float latency;
  int maxComms;
  int maxRecvs;
} ncclNetProperties_v6_t;

typedef struct {  /* src/extern/nccl_net.h:24-37 */
  char* name;
  char* pciPath;
  uint64_t guid;
  int ptrSupport;
  int speed;
  int port;
  float latency;
  int maxComms;
  int maxRecvs;
  ncclNetDeviceType netDeviceType;
  int netDeviceVersion;
} ncclNetProperties_v7_t;

typedef struct {
  char* name;
  char* pciPath;
  uint64_t guid;
  int ptrSupport;
  int regIsGlobal;  /* regMr is not tied to a particular comm */
  int speed;
  int port;
  float latency;
  int maxComms;
  int maxRecvs;
  ncclNetDeviceType netDeviceType;
  int netDeviceVersion;
} ncclNetProperties_v8_t;

/* ---- function tables ------------------------------------------------------------------------- */
typedef struct {  /* src/extern/nccl_net.h:118-163 */
  const char* name;
  ncclResult_t (*init)(ncclDebugLogger_t logFunction);
  ncclResult_t (*devices)(int* ndev);
  ncclResult_t (*getProperties)(int dev, ncclNetProperties_v6_t* props);
  ncclResult_t (*listen)(int dev, void* handle, void** listenComm);
  ncclResult_t (*connect)(int dev, void* handle, void** sendComm);
  ncclResult_t (*accept)(void* listenComm, void** recvComm);
  ncclResult_t (*regMr)(void* comm, void* data, int size, int type, void** mhandle);
  ncclResult_t (*regMrDmaBuf)(void* comm, void* data, size_t size, int type, uint64_t offset, int fd, void** mhandle);
  ncclResult_t (*deregMr)(void* comm, void* mhandle);
  ncclResult_t (*isend)(void* sendComm, void* data, int size, int tag, void* mhandle, void** request);
  ncclResult_t (*irecv)(void* recvComm, int n, void** data, int* sizes, int* tags, void** mhandles, void** request);
  ncclResult_t (*iflush)(void* recvComm, int n, void** data, int* sizes, void** mhandles, void** request);
  ncclResult_t (*test)(void* request, int* done, int* sizes);
  ncclResult_t (*closeSend)(void* sendComm);
  ncclResult_t (*closeRecv)(void* recvComm);
  ncclResult_t (*closeListen)(void* listenComm);
} ncclNet_v6_t;

typedef struct {  /* src/extern/nccl_net.h:41-94; instance at src/plugin.cc:1997-2017 */
  const char* name;
  ncclResult_t (*init)(ncclDebugLogger_t logFunction);
  ncclResult_t (*devices)(int* ndev);
  ncclResult_t (*getProperties)(int dev, ncclNetProperties_v7_t* props);
  ncclResult_t (*listen)(int dev, void* handle, void** listenComm);
  ncclResult_t (*connect)(int dev, void* handle, void** sendComm, ncclNetDeviceHandle_v7_t** sendDevComm);
  ncclResult_t (*accept)(void* listenComm, void** recvComm, ncclNetDeviceHandle_v7_t** recvDevComm);
  ncclResult_t (*regMr)(void* comm, void* data, int size, int type, void** mhandle);
  ncclResult_t (*regMrDmaBuf)(void* comm, void* data, size_t size, int type, uint64_t offset, int fd, void** mhandle);
  ncclResult_t (*deregMr)(void* comm, void* mhandle);
  ncclResult_t (*isend)(void* sendComm, void* data, int size, int tag, void* mhandle, void** request);
  ncclResult_t (*irecv)(void* recvComm, int n, void** data, int* sizes, int* tags, void** mhandles, void** request);
  ncclResult_t (*iflush)(void* recvComm, int n, void** data, int* sizes, void** mhandles, void** request);
  ncclResult_t (*test)(void* request, int* done, int* sizes);
  ncclResult_t (*closeSend)(void* sendComm);
  ncclResult_t (*closeRecv)(void* recvComm);
  ncclResult_t (*closeListen)(void* listenComm);
  ncclResult_t (*getDeviceMr)(void* comm, void* mhandle, void** dptr_mhandle);   /* NULL, as src/plugin.cc:2015 */
  ncclResult_t (*irecvConsumed)(void* recvComm, int n, void* request);          /* NULL, as src/plugin.cc:2016 */
} ncclNet_v7_t;

typedef struct {
  const char* name;
  ncclResult_t (*init)(ncclDebugLogger_t logFunction);
  ncclResult_t (*devices)(int* ndev);
  ncclResult_t (*getProperties)(int dev, ncclNetProperties_v8_t* props);
  ncclResult_t (*listen)(int dev, void* handle, void** listenComm);
  ncclResult_t (*connect)(int dev, void* handle, void** sendComm, ncclNetDeviceHandle_v8_t** sendDevComm);
  ncclResult_t (*accept)(void* listenComm, void** recvComm, ncclNetDeviceHandle_v8_t** recvDevComm);
  ncclResult_t (*regMr)(void* comm, void* data, size_t size, int type, void** mhandle);
  ncclResult_t (*regMrDmaBuf)(void* comm, void* data, size_t size, int type, uint64_t offset, int fd, void** mhandle);
  ncclResult_t (*deregMr)(void* comm, void* mhandle);
  ncclResult_t (*isend)(void* sendComm, void* data, int size, int tag, void* mhandle, void** request);
  ncclResult_t (*irecv)(void* recvComm, int n, void** data, int* sizes, int* tags, void** mhandles, void** request);
  ncclResult_t (*iflush)(void* recvComm, int n, void** data, int* sizes, void** mhandles, void** request);
  ncclResult_t (*test)(void* request, int* done, int* sizes);
  ncclResult_t (*closeSend)(void* sendComm);
  ncclResult_t (*closeRecv)(void* recvComm);
  ncclResult_t (*closeListen)(void* listenComm);
  ncclResult_t (*getDeviceMr)(void* comm, void* mhandle, void** dptr_mhandle);
  ncclResult_t (*irecvConsumed)(void* recvComm, int n, void* request);
} ncclNet_v8_t;

/* the data symbols a communication library resolves with dlsym() */
extern ncclNet_v8_t ncclNetPlugin_v8;
extern ncclNet_v7_t ncclNetPlugin_v7;
extern ncclNet_v6_t ncclNetPlugin_v6;

/* ---- limits restated from the reference -------------------------------------------------------- */
#define FL_NET_MAX_RECVS        8     /* NCCL_NET_IB_MAX_RECVS, src/plugin.cc:358 */
#define FL_NET_MAX_REQUESTS     256   /* MAX_REQUESTS = 32 * 8, src/plugin.cc:382 */
#define FL_NET_REFRESH_BATCH    8     /* N_FINISHED_BATCH, src/plugin.cc:38 */
#define FL_NET_MAX_LANES        16    /* MAX_NIC_NUM, src/monitor.h:18 */
#define FL_NET_MONITOR_TIMEOUT_US 160 /* MONITOR_TIMEOUT_US, src/monitor.h:26 */

/* ---- control surface beside the plugin tables (for a harness or a host runtime) ------------------
 * None of this is needed to use the plugin; it exposes what the reference keeps in its monitor
 * daemon's shared memory (src/monitor.h:47-55) and a few counters.  All return 0 or a negative
 * FLH_E_* code (fuselink_hip.h). */

/* Monitor state machine of src/monitor.h:191-250 and src/monitor.cpp:159-193, in-process, with the
 * clock passed in so that it is deterministic: mark = (timestamp, BUSY); tick = every NIC whose
 * timestamp + 160 us <= now becomes IDLE; pick = borrow an idle NIC of another group. */
int fl_monitor_reset(void);
/* Move the table into POSIX shared memory guarded by a named semaphore, the reference's arrangement
 * (src/monitor.h:23-24, 47-55; NULL names = "/rdma_monitor_shm", "/rdma_monitor_sem").  create = 1
 * makes and owns the objects (the daemon's part), create = 0 attaches to existing ones as the
 * reference's MonitorClient constructor does (src/monitor.h:110-133) and fails with FLH_E_STATE when
 * they are absent.  The layout is the reference's SharedMemory, so its client and this library can
 * share one table.  fl_monitor_detach returns to the process-local table. */
int fl_monitor_attach_shm(const char* shm_name, const char* sem_name, int create);
int fl_monitor_detach(void);
int fl_monitor_is_shared(void);
int fl_monitor_daemon_running(void);
/* Clock of the plugin's own marks and ticks: manual = 0 (default) reads the steady clock as
 * get_timestamp() does (src/monitor.h:29-33); manual = 1 freezes it at now_us until the next call,
 * which makes every lane decision reproducible. */
int fl_monitor_set_clock(int manual, int64_t now_us);
int64_t fl_monitor_now(void);
int fl_monitor_mark_active(int lane, int is_tx, int64_t now_us);
/* raw write of one table entry, as any process mapping the reference's shared memory could do */
int fl_monitor_set_entry(int lane, int is_tx, int32_t status, int64_t last_active_us);
int fl_monitor_tick(int64_t now_us);
int fl_monitor_status(int is_tx, int n_lanes, int32_t* status_out);
/* getIdleNicTx / getIdleNicRx (src/monitor.h:191-224).  `exact` = 0 restates the reference as
 * written (every idle NIC met is marked BORROWED and the last one is returned); `exact` = 1 borrows
 * only the first idle NIC, which is what the code evidently meant. */
int fl_monitor_idle_pick(int is_tx, int group, int mask, int exact);
/* Returns a BORROWED lane to IDLE at once (1 if it was borrowed, 0 if not): the release the reference
 * lacks, where a borrowed NIC only comes back through the daemon's ageing (src/monitor.cpp:171-186). */
int fl_monitor_release(int lane, int is_tx);
/* credits the scheduler will use from the next refresh on: IDLE -> idle_credit, BUSY/BORROWED -> 0,
 * the comm's own lane never below 1 */
int fl_monitor_credits(int n_lanes, int own_lane, uint32_t idle_credit, uint32_t* credits_out);
/* The two halves of the lane decision as the plugin takes it.  The sender's half: the usage mask that travels with its
 * data as imm_data (refreshTxUsage, src/fuselink.h:261-267, a placeholder there; src/plugin.cc:1441-1447, 1463) -- bit l
 * set when lane l's send side is IDLE in this host's table, the comm's own lane always, every bit from n_lanes on.  The
 * receiver's half, at its refresh (src/plugin.cc:1710; the mask of getIdleNicRx, src/monitor.h:208-224): idle_credit
 * for a lane whose receive side is IDLE here and that tx_mask admits, 0 otherwise, the own lane never below 1. */
int fl_monitor_tx_mask(int n_lanes, int own_lane, uint32_t* mask_out);
int fl_monitor_rx_credits(int n_lanes, int own_lane, uint32_t idle_credit, uint32_t tx_mask, uint32_t* credits_out);

/* Static credits (one value per lane) overriding the monitor-derived ones; n = 0 removes the
 * override.  The same can be preset with NCCL_FUSELINK_CREDITS="c0,c1,...". */
int fl_net_set_credits(const uint32_t* credits, int n);
/* Forget the parameters read at init so that the next init() reads the NCCL_FUSELINK_* environment
 * again; refused (FLH_E_STATE) while a listen comm or a connection is alive. */
int fl_net_reset(void);
/* Make the next completion of `request` fail in test() with ncclRemoteError (wire-fault injection). */
int fl_net_inject_fault(void* request);
/* Counters of a send or recv comm: n_finished (src/plugin.cc:517,568), requests in flight, lane refreshes. */
int fl_net_comm_stats(void* comm, int64_t* n_finished, int64_t* in_flight, int64_t* refreshes);
/* The lane-availability mask of a connection.  On a send comm: the mask it ships with its requests (imm_data of
 * src/plugin.cc:1463; getTxUsage / refreshTxUsage, src/fuselink.h:261-267) and how often it has been refreshed, which
 * happens before every send for which (n_finished + 1) % N_FINISHED_BATCH == 0 (src/plugin.cc:1443).  On a recv comm: the
 * mask that came with the latest completed receive (comm->txAvailable, src/plugin.cc:1884-1885), which its next refresh
 * ANDs into the credit row (src/plugin.cc:1710), and the number of lane refreshes. */
int fl_net_mask_stats(void* comm, uint32_t* mask, int64_t* refreshes);
/* Free slots of the comm's request table (256 when nothing is in flight, src/plugin.cc:382, 1070-1090). */
int fl_net_free_requests(void* comm);
/* Launch pairs (stripe + reassemble) that carried requests of the connection so far, and how many of its requests
 * travelled in a pair shared with other requests (its own or another connection's).  Matched sends of all connections
 * that stage on one GPU wait in one queue until a test() finds fewer than two launches queued on that GPU, or until
 * NCCL_FUSELINK_BATCH (default 32, 1 = launch inside isend) of them wait, then go out together. */
int fl_net_launch_stats(void* comm, int64_t* launches, int64_t* batched_requests);
/* Chunk -> lane rows of the connection's latest segment and the header of the launch that carried it, copied to host
 * memory (launches what waits and blocks until the GPU's queue has run).  rows_out holds up to max_rows
 * flh_chunk_desc entries.  Returns the number of rows of that segment; FLH_E_STATE if a later launch that did not
 * carry this connection has reused the table. */
int fl_net_last_table(void* sendComm, void* rows_out, int max_rows, void* hdr_out);
/* The last launch pair of the GPU that `comm` stages on: its segments (which connection, which rows of the table, how
 * many requests, where the connection stood in its credit epoch, where the segment starts in every lane's window),
 * the whole table and the header.  Returns the number of segments. */
typedef struct fl_net_launch_seg {
  int32_t channel;             /* channel id of the connection (src/plugin.cc:693-708) */
  uint32_t first_row, n_rows;  /* the segment's rows in the launch's table */
  uint32_t n_req;
  uint64_t epoch_bytes;        /* bytes of the connection's credit epoch before the segment */
  uint64_t lane_base[FL_NET_MAX_LANES];
} fl_net_launch_seg;
int fl_net_last_launch(void* comm, fl_net_launch_seg* segs_out, int max_segs, void* rows_out, int max_rows, void* hdr_out);
/* Where the host's time goes (collected only under NCCL_FUSELINK_TRACE=1; process-wide sums over all threads): calls
 * and nanoseconds, index 0 isend, 1 irecv, 2 test, 3 tests that completed a request (calls only), 4 passes that
 * launched what waited, 5 launch pairs (time inside the runtime's launch calls and the batch arithmetic before them),
 * 6 requests those passes launched (calls only), 7 batches handed to the lane engine (time inside flh_engine_submit),
 * 8 of those hand-overs that had to start the resident kernel first (counted apart from 7).  Returns the number of
 * counters. */
int fl_net_host_stats(int64_t* calls_out, int64_t* ns_out, int n);
/* Timeline kept under NCCL_FUSELINK_TRACE=2: up to 65536 events of 24 bytes {int64 nanoseconds (monotonic clock), uint32
 * thread, uint32 event, uint64 value}; events: 1 receive posted (value = channel), 2 send matched (channel), 3 a pass that
 * launches begins (requests waiting), 4 batch handed over (requests << 32 | bit 31: engine batch | its number),
 * 5 request seen complete by test (its batch's number << 16 | bit 15: an engine batch | channel << 1 | is-receive), 6 the
 * engine's batches seen complete up to this number, 7 wave announced to the receiving process (its number), 8 wave taken
 * off the wire by the receiving process (its number).  The clock is the same for every process of the machine.  Copies up
 * to max_events into `out`, returns how many exist. */
int fl_net_timeline(void* out, int max_events);
/* Launch whatever waits on the GPU that `comm` stages on, without polling a request. */
int fl_net_flush(void* comm);

#ifdef __cplusplus
}
#endif
#endif /* FUSELINK_NET_H_ */
