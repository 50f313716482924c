// fl_closed_form.h -- the schedule's closed form for quantum-sized chunks under one credit row, as host arithmetic.
// The copy kernels evaluate the same expressions per chunk on the GPU; the host needs the per-lane totals before a
// launch, to size a wave and to place the segments of a batch in the staging windows.
//
// Under a row of credits c_0 .. c_{L-1} (sum W; a row without any credit stands for equal credits, the round robin of
// FuseLink's static policy, src/fuselink.h:235) quantum x of a credit epoch takes slot x mod W, and lane l owns the
// slots [K_l, K_l + c_l), K_l the exclusive prefix of the row.  So the quanta before x that lane l received are
//     before(l, x) = (x / W) * c_l + clamp(x mod W - K_l, 0, c_l).
#ifndef FL_CLOSED_FORM_H_
#define FL_CLOSED_FORM_H_

#include <stdint.h>

#include "fuselink_hip.h"

struct FlCreditRow {
  uint64_t K[FLH_MAX_LANES + 1];   // exclusive prefixes; K[l] = W for l >= lanes
  uint64_t W;
  uint32_t lanes;
  bool zero;                       // the row had no credit: equal credits stand in (FLH_SCHED_F_NO_CREDIT)
};

inline void fl_row_make(const uint32_t* credits, uint32_t lanes, FlCreditRow& r) {
  uint64_t W = 0;
  for (uint32_t l = 0; l < lanes; ++l) W += credits[l];
  r.zero = W == 0;
  r.lanes = lanes;
  uint64_t run = 0;
  for (uint32_t l = 0; l <= FLH_MAX_LANES; ++l) {
    r.K[l] = run;
    if (l < lanes) run += r.zero ? 1 : credits[l];
  }
  r.W = run;
}

inline uint64_t fl_row_before(const FlCreditRow& r, uint32_t l, uint64_t x) {
  const uint64_t K = r.K[l], c = r.K[l + 1] - K;
  const uint64_t rem = x % r.W;
  return (x / r.W) * c + (rem <= K ? 0 : (rem - K < c ? rem - K : c));
}

inline uint32_t fl_row_lane_of(const FlCreditRow& r, uint64_t x) {
  const uint64_t slot = x % r.W;
  uint32_t lane = 0;
  for (uint32_t l = 0; l + 1 < r.lanes; ++l)
    if (r.K[l + 1] <= slot) lane = l + 1;
  return lane;
}

// Bytes and chunks that a message of `bytes` bytes in chunks of `chunk` puts on each lane when `quanta_before` quanta
// of its credit epoch precede it (only the last chunk may be short).  The two divisions by W are done once, not per
// lane: this runs for every request that waits for a launch.
inline void fl_row_lane_totals(const FlCreditRow& r, uint64_t quanta_before, uint64_t bytes, uint64_t chunk, uint64_t* lane_bytes,
                               uint32_t* lane_chunks) {
  const uint64_t n = (bytes + chunk - 1) / chunk;
  const uint64_t W = r.W, x0 = quanta_before, x1 = quanta_before + n;
  const uint64_t q0 = x0 / W, r0 = x0 - q0 * W, q1 = x1 / W, r1 = x1 - q1 * W;
  const uint32_t lanes = r.lanes;
  uint32_t last_lane = 0;
  const uint64_t last_slot = r1 ? r1 - 1 : W - 1;   // slot of quantum x1 - 1
  for (uint32_t l = 0; l < FLH_MAX_LANES; ++l) {
    uint64_t k = 0;
    if (l < lanes && n) {
      const uint64_t K = r.K[l], c = r.K[l + 1] - K;
      const uint64_t b1 = q1 * c + (r1 <= K ? 0 : (r1 - K < c ? r1 - K : c));
      const uint64_t b0 = q0 * c + (r0 <= K ? 0 : (r0 - K < c ? r0 - K : c));
      k = b1 - b0;
      if (l + 1 < lanes && r.K[l + 1] <= last_slot) last_lane = l + 1;
    }
    lane_chunks[l] = (uint32_t)k;
    lane_bytes[l] = k * chunk;
  }
  if (n) lane_bytes[last_lane] -= n * chunk - bytes;
}

#endif  // FL_CLOSED_FORM_H_
