// engine_bench.cc -- latency and rate of the lane engine (flh_engine_*) for batches of 512 KiB requests, without the
// plugin around it: what a batch costs one at a time, what it costs with several in flight, and what a submit costs
// that has to start the resident kernel again.  dlopen()s the library and prints one JSON line.
//
//   engine_bench <lib.so> [--requests N] [--depth D] [--workgroups W] [--batches B] [--span-mib S] [--trace 1] [--share1-tiles T]
// N requests per batch (1..32), D window sets = batches in flight (1..8), W workgroups of the engine (0 = default).
// --trace 1 (needs NCCL_FUSELINK_TEST_HOOKS=1): the engine stamps every batch's stages with the GPU's wall clock; a second
// JSON line gives the median time between consecutive stamps, for the batches that ran one at a time and for those
// that ran `depth` at a time, beside the host's submit -> completion seen for the same batches.
#include <dlfcn.h>
#include <hip/hip_runtime.h>

#include <algorithm>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <thread>
#include <vector>

#include "fuselink_hip.h"

#define HIP(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { fprintf(stderr, "%s -> %s\n", #x, hipGetErrorString(e_)); exit(3); } } while (0)
static double now_us() { return std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now().time_since_epoch()).count(); }

int main(int argc, char** argv) {
  if (argc < 2) { fprintf(stderr, "usage: %s <libnccl-net-fuselink.so> [--requests N] [--depth D] [--workgroups W] [--batches B] [--span-mib S]\n", argv[0]); return 1; }
  int nreq = 8, depth = 2, wgs = 0, batches = 2000, span_mib = 0, trace = 0, share1 = -1;
  for (int i = 2; i + 1 < argc; i += 2) {
    const std::string a = argv[i];
    const int v = atoi(argv[i + 1]);
    if (a == "--requests") nreq = v; else if (a == "--depth") depth = v; else if (a == "--workgroups") wgs = v; else if (a == "--batches") batches = v; else if (a == "--span-mib") span_mib = v; else if (a == "--trace") trace = v; else if (a == "--share1-tiles") share1 = v;
  }
  if (nreq < 1 || nreq > FLH_BATCH_MAX || depth < 1 || depth > 8 || batches < 1) { fprintf(stderr, "arguments out of range\n"); return 1; }
  void* lib = dlopen(argv[1], RTLD_NOW | RTLD_LOCAL);
  if (!lib) { fprintf(stderr, "dlopen: %s\n", dlerror()); return 1; }
#define SYM(name) decltype(&name) p_##name = (decltype(&name))dlsym(lib, #name); if (!p_##name) { fprintf(stderr, "missing %s\n", #name); return 1; }
  SYM(flh_init) SYM(flh_last_error) SYM(flh_engine_create) SYM(flh_engine_submit) SYM(flh_engine_completed) SYM(flh_engine_error) SYM(flh_engine_launches) SYM(flh_engine_destroy) SYM(flh_engine_needs_start) SYM(flh_engine_poke) SYM(flh_engine_trace) SYM(flh_tune)
  HIP(hipSetDevice(0));
  if (p_flh_init(0)) { fprintf(stderr, "init: %s\n", p_flh_last_error()); return 1; }
  const size_t req = 512 << 10, lanes = 8, cap = 4 << 20;
  // --span-mib S: successive batches walk through S MiB of sources and destinations, so that what a batch touches is in
  // no cache (the plugin's traffic); without it every batch moves the same buffers
  const size_t batch_bytes = req * nreq;
  const size_t slots = span_mib > 0 ? (((size_t)span_mib << 20) / batch_bytes ? ((size_t)span_mib << 20) / batch_bytes : 1) : 1;
  const size_t span = slots * batch_bytes;
  uint8_t *src, *dst, *win;
  HIP(hipMalloc((void**)&src, span)); HIP(hipMalloc((void**)&dst, span)); HIP(hipMalloc((void**)&win, (size_t)depth * lanes * cap));
  std::vector<uint8_t> pattern(span);
  uint64_t x = 88172645463325252ull;
  for (size_t i = 0; i < span; i += 8) { x ^= x << 13; x ^= x >> 7; x ^= x << 17; memcpy(&pattern[i], &x, 8); }
  HIP(hipMemcpy(src, pattern.data(), pattern.size(), hipMemcpyHostToDevice));
  HIP(hipMemset(dst, 0, span));
  flh_chunk_desc* table; flh_sched_hdr* hdr;
  HIP(hipMalloc((void**)&table, 4096 * sizeof(flh_chunk_desc))); HIP(hipMalloc((void**)&hdr, sizeof(flh_sched_hdr)));
  int32_t *h_status, *d_status;
  HIP(hipHostMalloc((void**)&h_status, 64, hipHostMallocMapped)); memset(h_status, 0, 64);
  HIP(hipHostGetDevicePointer((void**)&d_status, h_status, 0));
  std::vector<flh_windows> w(depth);
  for (int h = 0; h < depth; ++h) { memset(&w[h], 0, sizeof(flh_windows)); w[h].n_lanes = lanes; for (size_t l = 0; l < lanes; ++l) { w[h].base[l] = win + ((size_t)h * lanes + l) * cap; w[h].cap[l] = cap; } }
  flh_batch_params b; memset(&b, 0, sizeof(b));
  b.u.chunk_bytes = 256 << 10; b.u.n_lanes = lanes; b.u.tile_bytes = FLH_TILE_BYTES; b.u.total_bytes = (uint64_t)nreq * req;
  const uint32_t credits[8] = {8, 6, 7, 1, 8, 7, 3, 3};
  for (size_t l = 0; l < lanes; ++l) b.u.credits[l] = credits[l];
  b.n_req = nreq;
  for (int q = 0; q < nreq; ++q) b.bytes[q] = req;
  uint64_t submitted = 0;
  flh_engine* e = nullptr;
  if (share1 >= 0 && p_flh_tune("lane_share1_tiles", share1)) { fprintf(stderr, "tune: %s\n", p_flh_last_error()); return 1; }
  if (trace && p_flh_tune("engine_trace", 1)) { fprintf(stderr, "trace: %s\n", p_flh_last_error()); return 1; }
  if (trace && batches > 400) batches = 400;   // the engine keeps the stamps of its last 1024 batches
  if (p_flh_engine_create(0, wgs, 200, depth, &e)) { fprintf(stderr, "engine: %s\n", p_flh_last_error()); return 1; }
  uint64_t seq = 0;
  auto submit = [&](int set) {
    const size_t at = (size_t)(submitted++ % slots) * batch_bytes;
    for (int q = 0; q < nreq; ++q) { b.d_src[q] = src + at + q * req; b.d_dst[q] = dst + at + q * req; }
    if (p_flh_engine_submit(e, &b, &w[set], table, hdr, d_status, &seq, nullptr)) { fprintf(stderr, "submit: %s\n", p_flh_last_error()); exit(1); } };
  auto wait_for = [&](uint64_t upto) {
    const double deadline = now_us() + 5e6;
    while (p_flh_engine_completed(e) < upto) {
      // an engine whose time as a resident ran out leaves between two batches; whoever waits for one starts the next
      if (p_flh_engine_needs_start(e) && p_flh_engine_poke(e)) { fprintf(stderr, "poke: %s\n", p_flh_last_error()); exit(1); }
      if (now_us() > deadline) { fprintf(stderr, "timed out, engine error %d\n", p_flh_engine_error(e)); exit(2); }
    }
  };
  for (int i = 0; i < 10; ++i) { submit(i % depth); wait_for(seq); }
  // one batch at a time
  double t0 = now_us(), sub = 0;
  std::vector<double> host_alone;
  const uint64_t alone_first = seq + 1;
  for (int i = 0; i < batches; ++i) { const double a = now_us(); submit(i % depth); sub += now_us() - a; wait_for(seq); host_alone.push_back(now_us() - a); }
  const double alone = (now_us() - t0) / batches;
  const uint64_t piped_first = seq + 1;
  // `depth` batches in flight
  t0 = now_us();
  for (int i = 0; i < batches; ++i) { submit(i % depth); if (seq >= (uint64_t)depth) wait_for(seq - depth + 1); }
  wait_for(seq);
  const double piped = (now_us() - t0) / batches;
  // after the engine has gone down (idle for 1.5 ms)
  double restart_submit = 0, restart_done = 0;
  const int R = 20;
  for (int i = 0; i < R; ++i) {
    std::this_thread::sleep_for(std::chrono::microseconds(1500));
    const double a = now_us();
    submit(0);
    restart_submit += now_us() - a;
    wait_for(seq);
    restart_done += now_us() - a;
  }
  // the bytes must have arrived: every slot of the span that a batch has moved
  std::vector<uint8_t> back(span);
  HIP(hipMemcpy(back.data(), dst, span, hipMemcpyDeviceToHost));
  const size_t moved = (submitted < slots ? (size_t)submitted : slots) * batch_bytes;
  const bool exact = memcmp(back.data(), pattern.data(), moved) == 0 && h_status[0] == 0;
  printf("{\"harness\": \"engine\", \"requests_per_batch\": %d, \"request_bytes\": %zu, \"span_MiB\": %zu, \"window_sets\": %d, \"workgroups\": %d, \"batches\": %d, \"bit_exact\": %s, "
         "\"one_at_a_time_us_per_batch\": %.2f, \"submit_us\": %.2f, \"in_flight_us_per_batch\": %.2f, \"in_flight_us_per_request\": %.3f, \"in_flight_GBps_4N\": %.0f, "
         "\"after_idle_submit_us\": %.1f, \"after_idle_batch_us\": %.1f, \"engine_launches\": %llu}\n",
         nreq, req, span_mib > 0 ? span >> 20 : (size_t)0, depth, wgs, batches, exact ? "true" : "false", alone, sub / batches, piped, piped / nreq, 4.0 * nreq * req / (piped * 1e-6) / 1e9,
         restart_submit / R, restart_done / R, (unsigned long long)p_flh_engine_launches(e));
  if (trace) {
    // median ticks (10 ns) between consecutive stamps
    auto stages = [&](uint64_t first, uint32_t n, const char* name) {
      std::vector<uint64_t> st((size_t)n * FLH_ENGINE_STAMPS);
      if (p_flh_engine_trace(e, first, n, st.data())) { fprintf(stderr, "trace: %s\n", p_flh_last_error()); exit(1); }
      printf("\"%s\": {", name);
      static const char* const what[FLH_ENGINE_STAMPS] = {"", "tail_seen_to_published", "published_to_seen_by_first_worker", "seen_to_let_in", "let_in_to_descriptor_in_lds",
                                                          "descriptor_to_shares_moved_and_in_memory", "moved_to_completion_word_acknowledged"};
      for (int k = 1; k <= FLH_ENGINE_STAMPS; ++k) {
        std::vector<double> d;
        for (uint32_t i = 0; i < n; ++i) {
          const uint64_t a = st[(size_t)i * FLH_ENGINE_STAMPS + (k < FLH_ENGINE_STAMPS ? k - 1 : 0)], b = st[(size_t)i * FLH_ENGINE_STAMPS + (k < FLH_ENGINE_STAMPS ? k : FLH_ENGINE_STAMPS - 1)];
          if (a && b && b >= a) d.push_back((double)(b - a) / 100.0);
        }
        std::sort(d.begin(), d.end());
        printf("\"%s_us\": %.2f, ", k < FLH_ENGINE_STAMPS ? what[k] : "tail_seen_to_completion_word_acknowledged", d.empty() ? -1.0 : d[d.size() / 2]);
      }
      printf("\"batches\": %u}", n);
    };
    std::sort(host_alone.begin(), host_alone.end());
    printf("{\"harness\": \"engine_trace\", \"requests_per_batch\": %d, \"window_sets\": %d, \"host_submit_to_completion_seen_one_at_a_time_us\": %.2f, ", nreq, depth, host_alone[host_alone.size() / 2]);
    stages(alone_first, (uint32_t)batches, "one_at_a_time");
    printf(", ");
    stages(piped_first, (uint32_t)batches, "in_flight");
    printf("}\n");
  }
  p_flh_engine_destroy(e);
  return exact ? 0 : 5;
}
