// fl_vmm.cc -- staging windows on HIP virtual memory management.
//
// A pool holds `units` physical allocations of one staging unit each (2 MiB rounded up to the
// device's allocation granularity), created up front so that no physical allocation happens while
// traffic flows.  A window is a reserved virtual range; binding maps pool units behind its leading
// part, first free slot first (the slot policy of src/cumem.cu:157-175 in the FuseLink tree), and
// trimming returns them.  A region is the object built at memory-registration time: one window per
// lane for one user allocation, shared and reference counted by base address
// (src/plugin.cc:1212-1227, 1337-1408).
#include <hip/hip_runtime.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <new>
#include <vector>

#include "fl_internal.h"
#include "fuselink_hip.h"

#define FL_HIP(call)                                                                                        \
  do {                                                                                                      \
    hipError_t e_ = (call);                                                                                 \
    if (e_ != hipSuccess)                                                                                   \
      return fl_set_error(e_ == hipErrorNoDevice ? FLH_E_NODEV : FLH_E_HIP, "%s failed: %s (%s:%d)", #call, \
                          hipGetErrorString(e_), __FILE__, __LINE__);                                       \
  } while (0)

struct flh_pool {
  int device = 0;
  uint32_t units = 0;
  uint64_t gran = 0;
  uint64_t unit_bytes = 0;
  std::vector<hipMemGenericAllocationHandle_t> handle;
  std::vector<uint8_t> mapped;   // is_mapped of cumem.cu:16
  std::vector<void*> va;         // d_mem of cumem.cu:15
  int windows = 0;
  std::mutex mu;
};

struct flh_window {
  flh_pool* pool = nullptr;
  uint8_t* base = nullptr;
  uint64_t va_bytes = 0;
  std::vector<int> slots;        // slot backing unit k of the window
};

struct flh_region {
  flh_pool* pool = nullptr;
  uint8_t* base = nullptr;       // start_addr of FuseLinkMemHandle (src/fuselink.h:49)
  uint64_t bytes = 0;
  uint32_t n_lanes = 0;
  int nrefs = 0;                 // src/fuselink.h:44
  flh_window* win[FLH_MAX_LANES] = {};
};

namespace {
std::mutex g_region_mu;                      // addr2flmr_lock of src/plugin.cc:34
std::map<void*, flh_region*> g_regions;      // addr2flmr of src/plugin.cc:33

int64_t env_param(const char* name, int64_t dflt) {
  const char* v = getenv(name);
  if (!v || !*v) return dflt;
  char* end = nullptr;
  long long x = strtoll(v, &end, 0);
  return end && *end == 0 ? (int64_t)x : dflt;
}
}  // namespace

int64_t fl_param(const char* env_suffix, int64_t dflt) {
  char name[128];
  snprintf(name, sizeof(name), "NCCL_%s", env_suffix);
  return env_param(name, dflt);
}

extern "C" {

int flh_pool_create(int device, uint32_t units, flh_pool** out) {
  if (!out) return fl_set_error(FLH_E_ARG, "null out");
  *out = nullptr;
  if (units == 0 || units > 65536) return fl_set_error(FLH_E_ARG, "units %u out of range", units);
  int rc = flh_init(device);
  if (rc) return rc;
  flh_pool* p = new (std::nothrow) flh_pool();
  if (!p) return fl_set_error(FLH_E_NOMEM, "out of host memory");
  p->device = device;
  p->units = units;
  hipMemAllocationProp prop = {};
  prop.type = hipMemAllocationTypePinned;
  prop.location.type = hipMemLocationTypeDevice;
  prop.location.id = device;
  size_t gran = 0;
  hipError_t e = hipMemGetAllocationGranularity(&gran, &prop, hipMemAllocationGranularityMinimum);
  if (e != hipSuccess || gran == 0) {
    delete p;
    return fl_set_error(FLH_E_HIP, "hipMemGetAllocationGranularity failed: %s", hipGetErrorString(e));
  }
  p->gran = gran;
  // granularity is known before it is used (the reference divides by it while still zero,
  // src/fuselink.cc:15-18); the unit is 2 MiB rounded up to it (src/cumem.cu:50)
  p->unit_bytes = ((uint64_t)FLH_UNIT_BYTES + gran - 1) / gran * gran;
  p->handle.resize(units);
  p->mapped.assign(units, 0);
  p->va.assign(units, nullptr);
  for (uint32_t j = 0; j < units; ++j) {
    e = hipMemCreate(&p->handle[j], p->unit_bytes, &prop, 0);
    if (e != hipSuccess) {
      for (uint32_t k = 0; k < j; ++k) (void)hipMemRelease(p->handle[k]);
      delete p;
      return fl_set_error(FLH_E_HIP, "hipMemCreate of unit %u failed: %s", j, hipGetErrorString(e));
    }
  }
  *out = p;
  return FLH_OK;
}

int flh_pool_destroy(flh_pool* pool) {
  if (!pool) return FLH_OK;
  {
    std::lock_guard<std::mutex> g(pool->mu);
    if (pool->windows != 0) return fl_set_error(FLH_E_STATE, "%d windows still use the pool", pool->windows);
  }
  int rc = FLH_OK;
  for (uint32_t j = 0; j < pool->units; ++j) {
    hipError_t e = hipMemRelease(pool->handle[j]);
    if (e != hipSuccess) rc = fl_set_error(FLH_E_HIP, "hipMemRelease failed: %s", hipGetErrorString(e));
  }
  delete pool;
  return rc;
}

int flh_pool_free_units(const flh_pool* pool) {
  if (!pool) return fl_set_error(FLH_E_ARG, "null pool");
  flh_pool* p = const_cast<flh_pool*>(pool);
  std::lock_guard<std::mutex> g(p->mu);
  return (int)std::count(p->mapped.begin(), p->mapped.end(), (uint8_t)0);
}

int flh_pool_slot_of(const flh_pool* pool, const void* va) {
  if (!pool) return fl_set_error(FLH_E_ARG, "null pool");
  flh_pool* p = const_cast<flh_pool*>(pool);
  std::lock_guard<std::mutex> g(p->mu);
  for (uint32_t j = 0; j < p->units; ++j)
    if (p->mapped[j] && p->va[j] == va) return (int)j;
  return fl_set_error(FLH_E_ARG, "no unit is mapped at %p", va);
}

uint64_t flh_pool_granularity(const flh_pool* pool) { return pool ? pool->gran : 0; }

int flh_window_create(flh_pool* pool, uint64_t va_bytes, flh_window** out) {
  if (!pool || !out) return fl_set_error(FLH_E_ARG, "null argument");
  *out = nullptr;
  if (va_bytes == 0) return fl_set_error(FLH_E_ARG, "va_bytes must be > 0");
  flh_window* w = new (std::nothrow) flh_window();
  if (!w) return fl_set_error(FLH_E_NOMEM, "out of host memory");
  w->pool = pool;
  w->va_bytes = (va_bytes + pool->unit_bytes - 1) / pool->unit_bytes * pool->unit_bytes;  // src/fuselink.cc:29
  void* base = nullptr;
  hipError_t e = hipMemAddressReserve(&base, w->va_bytes, pool->unit_bytes, nullptr, 0);
  if (e != hipSuccess) {
    delete w;
    return fl_set_error(FLH_E_HIP, "hipMemAddressReserve(%llu) failed: %s", (unsigned long long)va_bytes, hipGetErrorString(e));
  }
  w->base = (uint8_t*)base;
  {
    std::lock_guard<std::mutex> g(pool->mu);
    pool->windows++;
  }
  *out = w;
  return FLH_OK;
}

int flh_window_bind(flh_window* w, uint64_t bytes) {
  if (!w) return fl_set_error(FLH_E_ARG, "null window");
  if (bytes > w->va_bytes) return fl_set_error(FLH_E_RANGE, "bind of %llu bytes exceeds the window's %llu", (unsigned long long)bytes, (unsigned long long)w->va_bytes);
  flh_pool* p = w->pool;
  const uint64_t need = (bytes + p->unit_bytes - 1) / p->unit_bytes;
  std::lock_guard<std::mutex> g(p->mu);
  while (w->slots.size() < need) {
    int slot = -1;
    for (uint32_t j = 0; j < p->units; ++j)
      if (!p->mapped[j]) { slot = (int)j; break; }
    if (slot < 0) return fl_set_error(FLH_E_NOMEM, "no free staging unit among %u", p->units);
    uint8_t* at = w->base + (uint64_t)w->slots.size() * p->unit_bytes;
    FL_HIP(hipMemMap(at, p->unit_bytes, 0, p->handle[slot], 0));
    hipMemAccessDesc acc = {};
    acc.location.type = hipMemLocationTypeDevice;
    acc.location.id = p->device;
    acc.flags = hipMemAccessFlagsProtReadWrite;
    hipError_t e = hipMemSetAccess(at, p->unit_bytes, &acc, 1);
    if (e != hipSuccess) {
      (void)hipMemUnmap(at, p->unit_bytes);
      return fl_set_error(FLH_E_HIP, "hipMemSetAccess failed: %s", hipGetErrorString(e));
    }
    p->mapped[slot] = 1;
    p->va[slot] = at;
    w->slots.push_back(slot);
  }
  return FLH_OK;
}

int flh_window_trim(flh_window* w, uint64_t bytes) {
  if (!w) return fl_set_error(FLH_E_ARG, "null window");
  flh_pool* p = w->pool;
  const uint64_t keep = (bytes + p->unit_bytes - 1) / p->unit_bytes;
  std::lock_guard<std::mutex> g(p->mu);
  while (w->slots.size() > keep) {
    const int slot = w->slots.back();
    uint8_t* at = w->base + (uint64_t)(w->slots.size() - 1) * p->unit_bytes;
    FL_HIP(hipMemUnmap(at, p->unit_bytes));
    p->mapped[slot] = 0;  // the reference's free_cumem leaves the flag set (src/cumem.cu:60-70)
    p->va[slot] = nullptr;
    w->slots.pop_back();
  }
  return FLH_OK;
}

int flh_window_destroy(flh_window* w) {
  if (!w) return FLH_OK;
  int rc = flh_window_trim(w, 0);
  if (rc) return rc;
  FL_HIP(hipMemAddressFree(w->base, w->va_bytes));
  {
    std::lock_guard<std::mutex> g(w->pool->mu);
    w->pool->windows--;
  }
  delete w;
  return FLH_OK;
}

void* flh_window_base(const flh_window* w) { return w ? w->base : nullptr; }

uint64_t flh_window_bound_bytes(const flh_window* w) { return w ? (uint64_t)w->slots.size() * w->pool->unit_bytes : 0; }

int flh_window_slots(const flh_window* w, int* slots, int max) {
  if (!w) return fl_set_error(FLH_E_ARG, "null window");
  std::lock_guard<std::mutex> g(w->pool->mu);
  for (int k = 0; k < max && k < (int)w->slots.size(); ++k) slots[k] = w->slots[k];
  return (int)w->slots.size();
}

int flh_window_export_dmabuf(const flh_window* w, uint64_t offset, uint64_t bytes, int* fd_out) {
  if (!w || !fd_out) return fl_set_error(FLH_E_ARG, "null argument");
  *fd_out = -1;
  const uint64_t unit = w->pool->unit_bytes;
  uint64_t bound;
  {
    std::lock_guard<std::mutex> g(w->pool->mu);
    bound = (uint64_t)w->slots.size() * unit;
  }
  // one descriptor covers one physical allocation, i.e. one unit (a longer range comes back truncated to its first unit)
  if (offset % unit || bytes != unit) return fl_set_error(FLH_E_ARG, "offset must be a multiple of the %llu-byte unit and bytes exactly one unit", (unsigned long long)unit);
  if (offset + bytes > bound) return fl_set_error(FLH_E_RANGE, "range %llu+%llu lies outside the %llu bound bytes", (unsigned long long)offset, (unsigned long long)bytes, (unsigned long long)bound);
  int fd = -1;
  FL_HIP(hipMemGetHandleForAddressRange(&fd, (hipDeviceptr_t)(w->base + offset), bytes, hipMemRangeHandleTypeDmaBufFd, 0));
  if (fd < 0) return fl_set_error(FLH_E_HIP, "no descriptor came back");
  struct stat st;
  if (fstat(fd, &st) != 0 || (uint64_t)st.st_size < bytes) {
    close(fd);
    return fl_set_error(FLH_E_HIP, "the descriptor covers less than the %llu bytes asked for", (unsigned long long)bytes);
  }
  *fd_out = fd;
  return FLH_OK;
}

int flh_region_acquire(flh_pool* pool, void* base, uint64_t bytes, uint32_t n_lanes, uint64_t bound_bytes_per_lane,
                       flh_region** out) {
  if (!pool || !base || !out) return fl_set_error(FLH_E_ARG, "null argument");
  *out = nullptr;
  if (bytes == 0) return fl_set_error(FLH_E_ARG, "bytes must be > 0");
  if (n_lanes > FLH_MAX_LANES) return fl_set_error(FLH_E_ARG, "n_lanes %u not in 0..%d", n_lanes, FLH_MAX_LANES);
  std::lock_guard<std::mutex> g(g_region_mu);
  auto it = g_regions.find(base);
  if (it != g_regions.end()) {  // src/plugin.cc:1214-1226: share the region, count the handle
    flh_region* r = it->second;
    if (r->n_lanes != n_lanes || r->pool != pool) return fl_set_error(FLH_E_STATE, "base %p is registered with another pool or lane count", base);
    r->nrefs++;
    *out = r;
    return FLH_OK;
  }
  flh_region* r = new (std::nothrow) flh_region();
  if (!r) return fl_set_error(FLH_E_NOMEM, "out of host memory");
  r->pool = pool;
  r->base = (uint8_t*)base;
  r->bytes = bytes;
  r->n_lanes = n_lanes;
  r->nrefs = 1;  // src/plugin.cc:1241
  for (uint32_t l = 0; l < n_lanes; ++l) {
    int rc = flh_window_create(pool, bytes, &r->win[l]);
    if (!rc) {
      uint64_t bind = std::min<uint64_t>(bound_bytes_per_lane, r->win[l]->va_bytes);
      rc = flh_window_bind(r->win[l], bind);
    }
    if (rc) {
      for (uint32_t k = 0; k <= l; ++k)
        if (r->win[k]) (void)flh_window_destroy(r->win[k]);
      delete r;
      return rc;  // message already set
    }
  }
  g_regions[base] = r;  // src/plugin.cc:1326
  *out = r;
  return FLH_OK;
}

int flh_region_release(flh_region* r) {
  if (!r) return fl_set_error(FLH_E_ARG, "null region");
  std::lock_guard<std::mutex> g(g_region_mu);
  if (r->nrefs <= 0) return fl_set_error(FLH_E_STATE, "region has no references");
  const int left = --r->nrefs;  // src/plugin.cc:1347
  if (left > 0) return left;
  g_regions.erase(r->base);     // src/plugin.cc:1398-1400
  int rc = FLH_OK;
  for (uint32_t l = 0; l < r->n_lanes; ++l) {
    int e = flh_window_destroy(r->win[l]);
    if (e) rc = e;
  }
  delete r;
  return rc;
}

int flh_region_refs(const flh_region* r) {
  if (!r) return fl_set_error(FLH_E_ARG, "null region");
  std::lock_guard<std::mutex> g(g_region_mu);
  return r->nrefs;
}

int flh_region_windows(const flh_region* r, flh_windows* out) {
  if (!r || !out) return fl_set_error(FLH_E_ARG, "null argument");
  memset(out, 0, sizeof(*out));
  out->n_lanes = r->n_lanes;
  for (uint32_t l = 0; l < r->n_lanes; ++l) {
    out->base[l] = r->win[l]->base;
    out->cap[l] = flh_window_bound_bytes(r->win[l]);
  }
  return FLH_OK;
}

void* flh_region_translate(const flh_region* r, uint32_t lane, const void* data) {
  if (!r || lane >= r->n_lanes) return nullptr;
  const uint8_t* d = (const uint8_t*)data;
  if (d < r->base || d >= r->base + r->bytes) return nullptr;
  return r->win[lane]->base + (d - r->base);  // src/plugin.cc:1582, 1626
}

}  // extern "C"
