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

#endif  // FL_INTERNAL_H_
