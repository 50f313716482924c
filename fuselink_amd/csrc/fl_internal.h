// fl_internal.h -- declarations shared by the translation units of libnccl-net-fuselink.so.
#ifndef FL_INTERNAL_H_
#define FL_INTERNAL_H_

#include <stdint.h>

// Stores a formatted message for flh_last_error() (thread-local) and returns `code`.
int fl_set_error(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

// NCCL_PARAM convention of the reference (src/extern/param.h:19-28): integer environment
// variables named NCCL_<NAME>, read once and cached.
int64_t fl_param(const char* env_suffix, int64_t dflt);

// Copy workgroups take their tiles in runs per XCD (xcd_tile() in fl_device.h): tiles per run and per block of 8 runs.
#ifndef FL_XCD_RUN_SHIFT
#define FL_XCD_RUN_SHIFT 5
#endif
constexpr uint32_t kXcdRunShift = FL_XCD_RUN_SHIFT;   // 32 tiles
constexpr uint32_t kXcdBlock = 8u << kXcdRunShift;    // 8 XCDs x 32 tiles

// Completion without a packet of its own: the next kernel the calling thread launches through the library carries
// `hip_event` as its completion event (hipEventQuery / hipEventSynchronize on it then answer for that kernel),
// which spares the barrier packet of a hipEventRecord behind it, during which the queue's next kernel does not
// start.  fl_completion_event_taken() says whether a launch took the event since it was handed over, and withdraws
// it if none did (nothing to launch, an error before the launch, or a profiling region is open and the launch
// carries that region's events): then record it the usual way.
__attribute__((visibility("hidden"))) void fl_completion_event(void* hip_event);
__attribute__((visibility("hidden"))) bool fl_completion_event_taken();

// Completion without any packet: the calling thread's next fused striping launch (flh_stripe_uniform,
// flh_stripe_batch) stores `value` to the host-visible word `d_word` from its first workgroup.  A kernel starts only
// once all earlier work of its stream has finished, so the word tells which launches are behind the queue's head.
// fl_launch_stamp_taken() says whether a launch took the stamp since it was handed over and withdraws it if none did.
__attribute__((visibility("hidden"))) void fl_launch_stamp(uint32_t* d_word, uint32_t value);
__attribute__((visibility("hidden"))) bool fl_launch_stamp_taken();

#endif  // FL_INTERNAL_H_
