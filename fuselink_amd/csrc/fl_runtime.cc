// fl_runtime.cc -- library state and the entry points that launch nothing: initialisation, the last error
// message, launch tunables, per-launch profiling, and the request -> QP split (host arithmetic).
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "fl_launch.h"

namespace {
thread_local char g_err[512] = "";

int64_t env_i64(const char* name, int64_t dflt) {
  const char* v = getenv(name);
  if (!v || !*v) return dflt;
  char* end = nullptr;
  long long x = strtoll(v, &end, 0);
  return end && *end == 0 ? x : dflt;
}
}  // namespace

int g_device = -1;
int g_cus = 0;
int g_grid_per_cu = 0;
int g_dest_order = -1;
int g_fused_fast = 1;
int g_nontemporal = -1;
int g_sched_variant = 0;
int g_sched_uniform_fast = 1;
int g_sched_seg_min = 4096;    // flh_tune("sched_seg_min"): chunks from which a workspace turns the scan into several workgroups
int g_copy_uniform_grid = 1;
int g_xcd_runs = 1;              // flh_tune("xcd_runs")
int64_t g_lane_share1_tiles = -1;  // flh_tune("lane_share1_tiles"): engine batches of up to this many copy tiles go out in one-tile shares (-1: three quarters of the workers)
int64_t g_engine_wait_us = 2000000;   // flh_tune("engine_wait_us"): limit of every wait inside a lane engine created afterwards
int g_engine_inject_fault = 0;        // flh_tune("engine_inject_fault"): an engine started while this is set fails at its first batch
int g_engine_trace = 0;               // flh_tune("engine_trace"): engines created afterwards keep wall-clock stamps of their batches (flh_engine_trace)
int g_engine_fail_start = 0;          // flh_tune("engine_fail_start"): starting an engine fails as if the launch had been refused

namespace {
thread_local ProfState t_prof;
}
ProfState& fl_prof() { return t_prof; }
int fl_set_error(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int fl_need_init() {
  if (g_device < 0) {
    int device = (int)env_i64("NCCL_FUSELINK_DEVICE", -1);
    if (device < 0 && hipGetDevice(&device) != hipSuccess) device = 0;   // unset: the caller's current device
    int rc = flh_init(device);
    if (rc) return rc;
  }
  return FLH_OK;
}

bool fl_use_nt(uint64_t working_set_bytes) {
  if (g_nontemporal >= 0) return g_nontemporal != 0;
  return working_set_bytes > kCacheResidentBytes;
}

int g_stream_force_deliver = -1;    // flh_tune("stream_mode_deliver"): -1 = from the two policies below
int g_stream_force[2] = {-1, -1};   // flh_tune("stream_mode_out" / "stream_mode_in"): -1 = the policy below

int fl_stream_mode(int dir, uint64_t bytes) {
  if (g_stream_force[dir] >= 0) return dir == 0 ? (g_stream_force[0] == 2 ? 3 : g_stream_force[0]) : (g_stream_force[1] == 1 ? 3 : g_stream_force[1]);
  if (g_nontemporal >= 0) return g_nontemporal ? 3 : 0;
  if (bytes > kWindowsCacheableBytes) return 3;               // the windows no longer fit the Infinity Cache
  if (dir == 0) return bytes >= (128ull << 20) ? 1 : 0;       // read the user buffer once, keep the windows cacheable
  return bytes >= (16ull << 20) ? 2 : 0;                      // windows come from cache; the user buffer is written past it
}

uint32_t fl_xcd_full(uint64_t grid) {
  if (!g_xcd_runs || grid < kXcdBlock || grid > 0xffffffffull) return 0;
  return ((uint32_t)grid & ~(kXcdBlock - 1)) | (g_xcd_runs == 2 ? 32u : 0u);   // (bit 5: each XCD an eighth of the grid, an experiment)
}

uint32_t fl_xcd_map(uint32_t width, uint32_t height) {
  if (width == 0 || (width & (width - 1)) || (uint64_t)width * height > 0xffffffffull) return 0;
  const uint32_t full = fl_xcd_full((uint64_t)width * height);
  if (full < kXcdBlock) return 0;
  uint32_t sh = 0;
  while ((1u << sh) < width) ++sh;
  return full | sh;   // full is a multiple of kXcdBlock >= 32, the shift stays below 32
}

uint32_t fl_copy_grid(uint64_t max_tiles) {
  uint64_t g = g_grid_per_cu > 0 ? (uint64_t)g_cus * (uint64_t)g_grid_per_cu : (1ull << 20);
  if (g > max_tiles) g = max_tiles;
  if (g < 1) g = 1;
  return (uint32_t)g;
}

extern "C" {

const char* flh_last_error(void) { return g_err; }

int64_t flh_constant(int which) {
  switch (which) {
    case 0: return FLH_TILE_BYTES;
    case 1: return FLH_MAX_LANES;
    case 2: return FLH_UNIT_BYTES;
    case 3: return FLH_POOL_UNITS;
    case 4: return sizeof(flh_chunk_desc);
    case 5: return sizeof(flh_sched_state);
    case 6: return sizeof(flh_sched_hdr);
    case 7: return 4;   // ABI version: 2 added flh_sched_params.d_table_by_lane, the batch entry points, the DMA-BUF export;
                        // 3 the per-tile descriptors (flh_sched_params.d_tiles, flh_stripe_tiles / flh_reassemble_tiles) and the fused paged pair;
                        // 4 batches of up to 32 requests in segments, the completion word / event in flh_uniform_params, flh_schedule_static
    case 8: return sizeof(flh_windows);
    case 9: return sizeof(flh_sched_params);
    case 10: return sizeof(flh_batch_params);
  }
  return -1;
}

int flh_init(int device) {
  int count = 0;
  hipError_t e = hipGetDeviceCount(&count);
  if (e != hipSuccess || count == 0)
    return fl_set_error(FLH_E_NODEV, "no HIP device: %s", e == hipSuccess ? "device count is 0" : hipGetErrorString(e));
  if (device < 0 || device >= count) return fl_set_error(FLH_E_ARG, "device %d out of range (%d devices)", device, count);
  FL_HIP(hipSetDevice(device));
  hipDeviceProp_t prop;
  FL_HIP(hipGetDeviceProperties(&prop, device));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return fl_set_error(FLH_E_NODEV, "device %d is %s; this library carries gfx950 code only", device, prop.gcnArchName);
  g_device = device;
  g_cus = prop.multiProcessorCount;
  g_grid_per_cu = (int)env_i64("NCCL_FUSELINK_GRID_PER_CU", g_grid_per_cu);
  g_nontemporal = (int)env_i64("NCCL_FUSELINK_NONTEMPORAL", g_nontemporal);
  if (g_grid_per_cu < 0) g_grid_per_cu = 0;
  return fl_sched_scratch_resolve(device);
}

int flh_prof_begin(int capacity) {
  if (capacity < 1 || capacity > (1 << 20)) return fl_set_error(FLH_E_ARG, "capacity %d out of range", capacity);
  if (!t_prof.ring) t_prof.ring = new std::vector<ProfRec>();
  while (t_prof.ring->size() < (size_t)capacity) {
    ProfRec r;
    r.kid = 0;
    FL_HIP(hipEventCreate(&r.e0));
    FL_HIP(hipEventCreate(&r.e1));
    t_prof.ring->push_back(r);
  }
  t_prof.n = 0;
  t_prof.on = true;
  return FLH_OK;
}

int flh_prof_end(double* us_out, int* kernel_out, int max) {
  t_prof.on = false;
  if (!t_prof.ring) return fl_set_error(FLH_E_STATE, "no profiling region was opened on this thread");
  const size_t n = t_prof.n;
  for (size_t i = 0; i < n; ++i) {
    ProfRec& r = (*t_prof.ring)[i];
    FL_HIP(hipEventSynchronize(r.e1));
    float ms = 0.f;
    FL_HIP(hipEventElapsedTime(&ms, r.e0, r.e1));
    if ((int)i < max) {
      if (us_out) us_out[i] = (double)ms * 1e3;
      if (kernel_out) kernel_out[i] = r.kid;
    }
  }
  t_prof.n = 0;
  return (int)n;
}

int flh_tune(const char* key, int64_t value) {
  if (!key) return fl_set_error(FLH_E_ARG, "null key");
  if (!strcmp(key, "grid_per_cu")) { if (value < 0) return fl_set_error(FLH_E_ARG, "grid_per_cu < 0"); g_grid_per_cu = (int)value; return FLH_OK; }
  if (!strcmp(key, "stripe_dest_order")) { g_dest_order = value < 0 ? -1 : (value != 0); return FLH_OK; }
  if (!strcmp(key, "fused_fast")) { g_fused_fast = value != 0; return FLH_OK; }
  if (!strcmp(key, "stream_mode_deliver")) {
    if (value < -1 || (value & ~19)) return fl_set_error(FLH_E_ARG, "%s: -1, or bits 0 (loads), 1 (stores that go on) and 4 (stores into the windows)", key);
    g_stream_force_deliver = (int)value;
    return FLH_OK;
  }
  if (!strcmp(key, "stream_mode_out") || !strcmp(key, "stream_mode_in")) {
    if (value < -1 || value > 3) return fl_set_error(FLH_E_ARG, "%s not in -1..3", key);
    g_stream_force[key[12] == 'i'] = (int)value;
    return FLH_OK;
  }
  if (!strcmp(key, "nontemporal")) { g_nontemporal = value < 0 ? -1 : (value != 0); return FLH_OK; }
  if (!strcmp(key, "xcd_runs")) { g_xcd_runs = value == 2 ? 2 : value != 0; return FLH_OK; }
  if (!strcmp(key, "lane_share1_tiles")) { g_lane_share1_tiles = value < 0 ? -1 : value; return FLH_OK; }
  if (!strncmp(key, "engine_", 7)) {
    // hooks for tests of the failure paths: a production process cannot reach them by accident
    const char* hooks = getenv("NCCL_FUSELINK_TEST_HOOKS");
    if (!hooks || strcmp(hooks, "1")) return fl_set_error(FLH_E_STATE, "%s is a test hook: set NCCL_FUSELINK_TEST_HOOKS=1 to use it", key);
    if (!strcmp(key, "engine_wait_us")) { if (value < 1) return fl_set_error(FLH_E_ARG, "engine_wait_us < 1"); g_engine_wait_us = value; return FLH_OK; }
    if (!strcmp(key, "engine_inject_fault")) { g_engine_inject_fault = value != 0; return FLH_OK; }
    if (!strcmp(key, "engine_fail_start")) { g_engine_fail_start = value != 0; return FLH_OK; }
    if (!strcmp(key, "engine_trace")) { g_engine_trace = value != 0; return FLH_OK; }
  }
  if (!strcmp(key, "copy_uniform_grid")) { g_copy_uniform_grid = value != 0; return FLH_OK; }
  if (!strcmp(key, "sched_seg_min")) {
    if (value < 1) return fl_set_error(FLH_E_ARG, "sched_seg_min < 1");
    g_sched_seg_min = (int)(value > 0x7fffffff ? 0x7fffffff : value);
    return FLH_OK;
  }
  if (!strcmp(key, "sched_uniform_fast")) { g_sched_uniform_fast = value != 0; return FLH_OK; }
  if (!strcmp(key, "sched_variant")) { if (value < 0 || value > 6) return fl_set_error(FLH_E_ARG, "sched_variant not in 0..6"); g_sched_variant = (int)value; return FLH_OK; }
  return fl_set_error(FLH_E_ARG, "unknown tunable %s", key);
}

int flh_qp_split(int size, int nqps, int* off, int* len) {
  if (nqps < 1 || size < 0 || !off || !len) return fl_set_error(FLH_E_ARG, "bad qp split arguments");
  // stride = ceil(ceil(size / nqps) / 128) * 128; a piece past the end is an empty work request.
  // 64-bit inside: the reference's `int` expression overflows for sizes within 127 bytes of INT_MAX.
  const int64_t per = ((int64_t)size + nqps - 1) / nqps;
  const int64_t stride = (per + 127) / 128 * 128;
  int64_t o = 0;
  for (int q = 0; q < nqps; ++q, o += stride) {
    int64_t l = (int64_t)size - o;
    if (l > stride) l = stride;
    off[q] = o > 0x7fffffff ? 0x7fffffff : (int)o;
    len[q] = l > 0 ? (int)l : 0;
  }
  return stride > 0x7fffff80 ? 0x7fffff80 : (int)stride;
}

}  // extern "C"
