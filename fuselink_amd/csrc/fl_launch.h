// fl_launch.h -- host-side state and helpers shared by the translation units that launch kernels: the launch
// tunables, the per-thread profiling ring behind flh_prof_begin / flh_prof_end, and the launch macro.
#ifndef FL_LAUNCH_H_
#define FL_LAUNCH_H_

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include <vector>

#include "fl_internal.h"
#include "fuselink_hip.h"

#define FL_LOCAL __attribute__((visibility("hidden")))

// device the library was initialised on and its compute-unit count (-1 / 0 before flh_init)
extern FL_LOCAL int g_device;
extern FL_LOCAL int g_cus;
// launch tunables (flh_tune; some can be preset through NCCL_FUSELINK_* for experiments)
extern FL_LOCAL int g_grid_per_cu;         // 0: one workgroup per tile (up to 2^20)
extern FL_LOCAL int g_dest_order;          // fused striping in destination order: -1 = when the working set exceeds the cache, 0 / 1 force
extern FL_LOCAL int g_fused_fast;          // host-prepared reciprocal for the fused kernels' slot arithmetic (0 = always divide in the kernel)
extern FL_LOCAL int g_nontemporal;         // -1: streaming accesses only when the buffers cannot all sit in the Infinity Cache
extern FL_LOCAL int g_sched_variant;       // 0 = pick the scheduler shape from the chunk count
extern FL_LOCAL int g_sched_uniform_fast;
extern FL_LOCAL int g_sched_seg_min;
extern FL_LOCAL int64_t g_engine_wait_us;
extern FL_LOCAL int g_engine_inject_fault;
extern FL_LOCAL int g_engine_fail_start;
extern FL_LOCAL int g_engine_trace;
extern FL_LOCAL int g_copy_uniform_grid;
extern FL_LOCAL int64_t g_lane_share1_tiles;
extern FL_LOCAL int g_stream_force_deliver;
extern FL_LOCAL int g_xcd_runs;            // copy workgroups take their tiles in runs per XCD (see xcd_tile)
constexpr uint64_t kCacheResidentBytes = 512ull << 20;  // plain copy: working sets up to this stay largely in the 256 MB Infinity Cache
constexpr uint64_t kWindowsCacheableBytes = 256ull << 20;  // a message whose staging windows still fit the Infinity Cache

// Per-launch timing: while a profiling region is open on the calling thread, every kernel is launched
// with its own start/stop events (hipExtLaunchKernelGGL), which bracket the kernel alone and not the
// gaps around it.  The events are read back when the region is closed, so the launches themselves
// stay asynchronous and back to back.
struct ProfRec { hipEvent_t e0, e1; int kid; };
struct ProfState {
  std::vector<ProfRec>* ring = nullptr;
  size_t n = 0;
  bool on = false;
  int kid = 0;   // which entry point is launching: 1 schedule, 2 stripe, 3 reassemble, 4 gather, 5 scatter, 6 copy
};
// The calling thread's state.  Reached through a function, not through an `extern thread_local`: code that uses
// such a variable from another translation unit tests the address of its (absent, weak, hidden) initialiser,
// which position-independent code computes relative to the load address, never as null, and then calls it.
FL_LOCAL ProfState& fl_prof();

// `ev` (may be null) is completed by the kernel itself; inside a profiling region the launch carries that region's
// events and `ev` is recorded behind it instead.
#define FL_LAUNCH_EV(kernel, grid, block, shmem, stream, ev, ...)                                       \
  do {                                                                                                  \
    ProfState& ps_ = fl_prof();                                                                         \
    hipEvent_t ev_ = (ev);                                                                              \
    if (ps_.on && ps_.n < ps_.ring->size()) {                                                           \
      ProfRec& pr_ = (*ps_.ring)[ps_.n++];                                                              \
      pr_.kid = ps_.kid;                                                                                \
      hipExtLaunchKernelGGL(kernel, grid, block, shmem, stream, pr_.e0, pr_.e1, 0, __VA_ARGS__);        \
      if (ev_) (void)hipEventRecord(ev_, stream);                                                       \
    } else if (ev_) {                                                                                   \
      hipExtLaunchKernelGGL(kernel, grid, block, shmem, stream, nullptr, ev_, 0, __VA_ARGS__);          \
    } else {                                                                                            \
      hipLaunchKernelGGL(kernel, grid, block, shmem, stream, __VA_ARGS__);                              \
    }                                                                                                   \
  } while (0)
#define FL_LAUNCH(kernel, grid, block, shmem, stream, ...) FL_LAUNCH_EV(kernel, grid, block, shmem, stream, (hipEvent_t) nullptr, __VA_ARGS__)

#define FL_HIP(call)                                                                         \
  do {                                                                                       \
    hipError_t e_ = (call);                                                                  \
    if (e_ != hipSuccess)                                                                    \
      return fl_set_error(e_ == hipErrorNoDevice ? FLH_E_NODEV : FLH_E_HIP, "%s failed: %s (%s:%d)", #call, \
                          hipGetErrorString(e_), __FILE__, __LINE__);                        \
  } while (0)

// flh_init on NCCL_FUSELINK_DEVICE (unset: the calling thread's current device) if no entry point has initialised the library yet
FL_LOCAL int fl_need_init();
// Non-temporal loads and stores pay off once the working set (the buffers a transfer touches) is well
// beyond the 256 MB Infinity Cache (measured: +3-5 % at 1 GiB messages) and cost throughput when a
// good part of it still fits (-8 % at 64 MiB, -20 % on the read-back side at 128 MiB).
FL_LOCAL bool fl_use_nt(uint64_t working_set_bytes);
// Streaming mode of a striping (dir 0) or reassembly (dir 1) launch that moves `bytes`: bit 0 = streaming loads,
// bit 1 = streaming stores.  What is used once streams -- the user buffer read by the striping side from 128 MiB
// on, the user buffer written by the reassembly side from 16 MiB on -- and the staging windows, written by one
// launch and read by the next, stay cacheable until they outgrow the 256 MB Infinity Cache (then everything
// streams; at 320 MiB the cacheable variant already thrashes: reassembly 146 instead of 117 us).  Measured
// against all-cached / all-streaming, stripe + reassemble over one pair of user buffers: 64 MiB equal, 96 MiB
// +4 %, 128 MiB +8 %, 192 MiB +11 %, 256 MiB +9 %, 384 MiB and beyond equal; over user buffers that no cache
// holds (pairs in rotation): 32 MiB +3 %, 64 MiB +4.5 %, 128 MiB +6 %.
FL_LOCAL int fl_stream_mode(int dir, uint64_t bytes);
// workgroups for a copy over max_tiles tiles: one per tile (the dispatcher then overlaps loads and stores of
// different tiles); the kernels' stride loops only matter beyond the cap, which grid_per_cu can lower
FL_LOCAL uint32_t fl_copy_grid(uint64_t max_tiles);

// xcd_tile()'s `full` for a one-dimensional grid, and xcd_tile_2d()'s map for a grid (width, height): 0 (off) unless the
// mapping is switched on, the grid has 256 workgroups or more and, for the latter, the width is a power of two below 2^32 / height.
FL_LOCAL uint32_t fl_xcd_full(uint64_t grid);
FL_LOCAL uint32_t fl_xcd_map(uint32_t width, uint32_t height);

// Resolves, once per device and with that device current, the address of the device's copy of the workspace that
// flh_schedule_static brings along (hipGetSymbolAddress); called by flh_init, and by the entry point's first call on
// any other device.
extern "C" FL_LOCAL int fl_sched_scratch_resolve(int device);

#endif  // FL_LAUNCH_H_
