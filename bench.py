#!/usr/bin/env python3
"""Benchmark of the FuseLink data path on one MI355X.

One step = the whole hot path over one message: chunk -> lane scheduling, striping (user buffer ->
per-lane HIP-VMM staging windows) and reassembly (windows -> receive buffer).  The default workload
is the headline configuration: a 64 MiB fp16 gradient-bucket buffer (N(0,1), seeded), 256 KiB chunks,
8 lanes, lane credits uniform in [1,8] (seeded).  Inputs are resident in HBM before the timed region.
Prints one JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--path auto|fused|split]
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0

WORKLOADS = {
    # name: (kind, bytes, chunk bytes, lanes, credit rows, epoch length)
    "cfg2_grad_bucket_64MiB_256KiB_8lanes": ("uniform", 64 << 20, 256 << 10, 8, 1, 0),
    "cfg5_stress_1GiB_64KiB_16lanes": ("uniform", 1 << 30, 64 << 10, 16, 17, 1000),
    # 256 variable blocks of 7168-wide bf16 rows, rows ~ Zipf(1.1) capped at 4096; the chunks are the blocks
    "cfg3_expert_parallel_256_blocks_8lanes": ("blocks", 0, 256 << 10, 8, 1, 0),
    # K and V pools of 4096 pages of 32 KiB each, seeded page permutation, 128 KiB chunks (4 pages)
    "cfg4_paged_kv_2x4096_pages_8lanes": ("pages", 2 * 4096 * 32768, 128 << 10, 8, 1, 0),
}

# Bytes per launch of the striping kernel between the L2 caches and the fabric behind them (Infinity Cache, then HBM),
# from two rocprofv3 --pmc runs (FETCH_SIZE, then WRITE_SIZE), each scaled by what the same counter reads for the plain
# copy kernel of known size.  None where no such run has been recorded for the workload.
MEASURED_TRAFFIC = {"cfg2_grad_bucket_64MiB_256KiB_8lanes": 134277565,
                    "cfg2_grad_bucket_64MiB_256KiB_8lanes/carry": 201425313, "cfg2_grad_bucket_64MiB_256KiB_8lanes/deliver": 201554230,
                    "cfg5_stress_1GiB_64KiB_16lanes": 2148014006,
                    "cfg5_stress_1GiB_64KiB_16lanes/17 waves": 126482128,
                    "cfg3_expert_parallel_256_blocks_8lanes": 1786029836, "cfg4_paged_kv_2x4096_pages_8lanes": 268579065}
# ... and the summary under profiles/ that each figure comes from (the counters are not read by this script: `traffic` is
# a recorded measurement of the same kernel on the same workload, the file holds the commands that made it)
TRAFFIC_SOURCE = {"cfg2_grad_bucket_64MiB_256KiB_8lanes": "profiles/copy_kernels_cfg2_l2_fabric_traffic.md",
                  "cfg2_grad_bucket_64MiB_256KiB_8lanes/carry": "profiles/copy_kernels_cfg2_l2_fabric_traffic.md",
                  "cfg2_grad_bucket_64MiB_256KiB_8lanes/deliver": "profiles/copy_kernels_cfg2_l2_fabric_traffic.md",
                  "cfg5_stress_1GiB_64KiB_16lanes": "profiles/copy_kernels_cfg5_l2_fabric_traffic.md",
                  "cfg5_stress_1GiB_64KiB_16lanes/17 waves": "profiles/copy_kernels_cfg5_l2_fabric_traffic.md",
                  "cfg3_expert_parallel_256_blocks_8lanes": "profiles/copy_kernels_cfg3_l2_fabric_traffic.md",
                  "cfg4_paged_kv_2x4096_pages_8lanes": "profiles/page_kernels_cfg4_l2_fabric_traffic.md"}


def algo_bytes_cold(nbytes: int) -> int:
    return 4 * nbytes   # stripe: read N + write N; reassemble: read N + write N


def _state_at(core, dev, epoch_bytes, chunk):
    """Scheduler state of a message of whole chunks that has `epoch_bytes` bytes of its one epoch behind it."""
    import numpy as np
    import torch
    st = np.zeros(1, dtype=core.STATE_DTYPE)
    st["epoch_bytes"], st["chunk_index"] = epoch_bytes, epoch_bytes // chunk
    return torch.from_numpy(st.view(np.uint8)).to(dev)


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="cfg2_grad_bucket_64MiB_256KiB_8lanes", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-iters", type=int, default=1000, help="timed CPU passes at 64 MiB (scaled down for larger messages): about 5 s of CPU work per figure")
    ap.add_argument("--hint", type=int, default=1, help="pass the host-known header fields to the copy kernels")
    ap.add_argument("--path", default="auto", choices=["auto", "fused", "split", "carry", "deliver"],
                    help="fused: scheduler folded into the striping launch (uniform split, one credit row); split: three launches; "
                         "carry: the launches of a transfer whose receiver is another process and has not exported its buffer -- the striping "
                         "launch also carries every staged tile into a second set of windows (the receiver's landing windows, here a plain "
                         "allocation of this process), the reassembly reads from those; deliver: the one launch of a transfer whose receive buffer the "
                         "sender can write itself -- staged into the windows and written into the destination from the same registers "
                         "(flh_stage_deliver_uniform; 3 x bytes per step instead of 4); neither is the bench line")
    ap.add_argument("--lds", type=int, default=0, help="paged workload: stage the gather through LDS")
    ap.add_argument("--cold-user-buffers", type=int, default=1,
                    help="also time the step over source/destination pairs in rotation (1 GiB), so that no user buffer is "
                         "cache-resident (fused uniform workloads up to 128 MiB); it runs after the timed loop and the per-kernel "
                         "passes, so a kernel trace of the run holds the timed loop's launches first; 0 = skip")
    ap.add_argument("--scheduler-bench", type=int, default=1,
                    help="also time the scheduler kernels on the stress configuration's chunk list (16384 chunks, 16 lanes, 17 credit "
                         "rows, epochs of 1000): closed form, scan on one workgroup, scan on a workgroup per 1024 chunks; 0 = skip")
    ap.add_argument("--plugin-bench", type=int, default=1,
                    help="also move the headline message through the plugin ABI in the shape a communication library drives it "
                         "(tests/harness/plugin_harness as a child process, started before this process touches the GPU): "
                         "128 requests of 512 KiB, 8 in flight, one connection and four; the same shape on 256 MiB per connection; "
                         "one batch of eight requests through the lane engine alone (tests/harness/engine_bench); 0 = skip")
    ap.add_argument("--ragged", action="store_true",
                    help="blocks workload: add 1..15 bytes to every block, so that no chunk is a multiple of 16 bytes and source and "
                         "window offsets are misaligned against each other")
    ap.add_argument("--tune", action="append", default=[], metavar="KEY=VALUE",
                    help="set a library tunable (flh_tune) before the run, e.g. --tune xcd_runs=0; repeatable")
    ap.add_argument("--blocks", type=int, default=256,
                    help="blocks workload: number of variable blocks (rows per block ~ Zipf(1.1) capped at 4096 for the 256 blocks of cfg3, "
                         "at 65536 / blocks otherwise: 65000 blocks are single rows of 14 KiB)")
    ap.add_argument("--tile-descriptors", type=int, default=-1,
                    help="blocks workload: let the scheduler expand the table to one descriptor per copy tile (flh_stripe_tiles); "
                         "-1 = when the blocks average under two copy tiles and there are at least 4096 of them")
    ap.add_argument("--cache-waves", type=int, default=-1,
                    help="uniform workloads past 256 MiB: move the message in waves small enough for the staging windows to stay in the "
                         "256 MB Infinity Cache (a wave is a credit epoch where the workload has epochs, else 64 MiB), each wave one fused "
                         "stripe + reassemble pair over the same windows; -1 = do so, 0 = one launch pair for the whole message")
    ap.add_argument("--wave-epochs", type=int, default=1,
                    help="workloads with credit epochs: epochs per cache-resident wave.  1 = a fused launch pair per epoch; more = one "
                         "scheduler launch for the whole message (wave_chunks) and a table-driven launch pair per wave")
    ap.add_argument("--pool-units", type=int, default=0,
                    help="uniform table-driven workloads: keep the staging windows within a pool of this many 2 MiB units (the reference's "
                         "holds 256) and move the message in as few waves as that allows, windows reused wave by wave; 0 = windows for the whole message")
    ap.add_argument("--lanes", type=int, default=0,
                    help="override the workload's number of lanes (staging windows); for measuring what the window count costs, not a bench line")
    ap.add_argument("--no-by-lane", action="store_true", help="stripe large messages in chunk order instead of destination order")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (every lane's staging window lives on it); "
              f"--gpus {args.gpus} is not supported", file=sys.stderr)
        return 2

    # ---- the plugin ABI, driven as a communication library drives it: a child process, before this one uses the GPU ----
    plugin = None
    if args.plugin_bench and args.workload.startswith("cfg2"):
        import subprocess

        from fuselink_amd import build as flbuild
        harness = os.path.join(ROOT, "tests", "harness", "plugin_harness")
        if os.path.exists(harness) and os.path.exists(flbuild.lib_path()):
            env = dict(os.environ, NCCL_FUSELINK_LANES="8", NCCL_FUSELINK_CHUNKSIZE=str(256 << 10))
            plugin = {"message_bytes": 64 << 20, "request_bytes": 512 << 10, "requests": 128, "inflight": 8, "lanes": 8, "chunk_bytes": 256 << 10,
                      "accounting": "4 x bytes x connections / wall time of the best of 20 iterations, proxy threads started inside the timed region.  4 x bytes is the headline metric's accounting (stage: read N + write N, deliver: read N + write N) and what a striping and a reassembly launch move; the plugin's engine batches and, by default, its launches load every vector once and store it twice (staging window and receive buffer) and so move 3 x bytes for the same result: payload rate = GBps_4N / 4",
                      "env": "NCCL_FUSELINK_LANES=8 NCCL_FUSELINK_CHUNKSIZE=262144"}
            for conns in (1, 4):
                cmd = [harness, flbuild.lib_path(), "--bytes", str(64 << 20), "--request", str(512 << 10), "--inflight", "8", "--iters", "20",
                       "--connections", str(conns)]
                try:
                    res = subprocess.run(cmd, capture_output=True, text=True, timeout=120, env=env)
                    line = json.loads(res.stdout.strip().splitlines()[-1]) if res.returncode == 0 else None
                except Exception:
                    line = None
                key = f"connections_{conns}"
                if line and line.get("bit_exact"):
                    plugin[key] = {"GBps_4N": line["GBps_4N_best"], "best_s": line["best_s"], "mean_s": line["mean_s"], "bit_exact": True,
                                   "us_per_request": round(line["best_s"] * 1e6 / (128 * conns), 3)}
                else:
                    plugin[key] = None
                plugin[key + "_command"] = " ".join(os.path.relpath(c, ROOT) if os.path.isabs(c) else c for c in cmd)
            # the same request shape on a message long enough (256 MiB per connection, 512 requests) for the threads' start
            # and the lane engine's to be a small part of an iteration: the rate the round trip of a request allows
            for conns in (1, 4):
                cmd = [harness, flbuild.lib_path(), "--bytes", str(256 << 20), "--request", str(512 << 10), "--inflight", "8", "--iters", "12",
                       "--connections", str(conns)]
                try:
                    res = subprocess.run(cmd, capture_output=True, text=True, timeout=120, env=env)
                    line = json.loads(res.stdout.strip().splitlines()[-1]) if res.returncode == 0 else None
                except Exception:
                    line = None
                key = f"long_message_256MiB_connections_{conns}"
                if line and line.get("bit_exact"):
                    plugin[key] = {"GBps_4N": line["GBps_4N_best"], "best_s": line["best_s"], "mean_s": line["mean_s"], "bit_exact": True,
                                   "us_per_request": round(line["best_s"] * 1e6 / (512 * conns), 3)}
                else:
                    plugin[key] = None
                plugin[key + "_command"] = " ".join(os.path.relpath(c, ROOT) if os.path.isabs(c) else c for c in cmd)
            # Sender and receiver in different processes (NCCL_FUSELINK_WIRE=shm; the harness forks the receiver before either
            # side has loaded the plugin or touched the GPU): NCCL's request shape, 64 MiB requests, and the five messages of
            # the serving experiment's KV hand-off.  Payload bytes over the wall time of the best iteration, as a user of the
            # connection sees it; "landing_windows" is the same shape with the receiver's registrations not exported.
            two = {"accounting": "payload bytes / wall time of the best iteration, measured in the sending process from its first isend to its last completed send",
                   "env": "NCCL_FUSELINK_LANES=8 NCCL_FUSELINK_CHUNKSIZE=262144 (the harness sets NCCL_FUSELINK_WIRE=shm)"}
            shapes = {
                "two_process_512KiB_x8_256MiB": (["--two-process", "--bytes", str(256 << 20), "--request", str(512 << 10), "--inflight", "8", "--iters", "10"], {}),
                "two_process_64MiB_x4_1GiB": (["--two-process", "--bytes", str(1 << 30), "--request", str(64 << 20), "--inflight", "4", "--iters", "6"], {}),
                "two_process_kv_handoff": (["--two-process", "--handoff", "8,64,4,8,16,128", "--request", str(512 << 10), "--inflight", "8", "--iters", "6"], {}),
                "two_process_512KiB_x8_256MiB_landing_windows": (["--two-process", "--bytes", str(256 << 20), "--request", str(512 << 10), "--inflight", "8", "--iters", "10"],
                                                                 {"NCCL_FUSELINK_WIRE_DIRECT": "0"}),
                "two_process_64MiB_x4_1GiB_landing_windows": (["--two-process", "--bytes", str(1 << 30), "--request", str(64 << 20), "--inflight", "4", "--iters", "6"],
                                                              {"NCCL_FUSELINK_WIRE_DIRECT": "0"}),
            }
            for key, (argv, extra) in shapes.items():
                cmd = [harness, flbuild.lib_path(), *argv]
                try:
                    res = subprocess.run(cmd, capture_output=True, text=True, timeout=180, env=dict(env, **extra))
                    line = json.loads(res.stdout.strip().splitlines()[-1]) if res.returncode == 0 else None
                except Exception:
                    line = None
                if line and line.get("bit_exact"):
                    two[key] = {"GBps_payload": line["GBps_payload_best"], "best_s": line["best_s"], "mean_s": line["mean_s"], "requests": line["requests"], "bit_exact": True}
                else:
                    two[key] = None
                two[key + "_command"] = " ".join([f"{k}={v}" for k, v in extra.items()] + [os.path.relpath(c, ROOT) if os.path.isabs(c) else c for c in cmd])
            plugin["two_process"] = two
            # The plugin beside an application's own streams: eight more streams of the process kept busy with small fills
            # while one connection moves 1 GiB at NCCL's request shape.  More streams than hardware queues, so some share a
            # queue with the plugin's: how long a fill takes from launch to completion shows how long the plugin's kernels
            # (the resident lane engine above all) hold a queue.
            cmd = [harness, flbuild.lib_path(), "--bytes", str(1 << 30), "--request", str(512 << 10), "--inflight", "8", "--iters", "3", "--side-streams", "8"]
            try:
                res = subprocess.run(cmd, capture_output=True, text=True, timeout=180, env=env)
                rows = {l["harness"]: l for l in (json.loads(x) for x in res.stdout.strip().splitlines() if x.startswith("{"))} if res.returncode == 0 else {}
            except Exception:
                rows = {}
            if rows.get("plugin", {}).get("bit_exact") and "side_streams" in rows:
                plugin["beside_8_busy_streams"] = {"GBps_4N": rows["plugin"]["GBps_4N_best"], "fills": rows["side_streams"]["fills"],
                                                   "fill_us_mean": rows["side_streams"]["fill_us_mean"], "fill_us_max": rows["side_streams"]["fill_us_max"], "bit_exact": True}
            else:
                plugin["beside_8_busy_streams"] = None
            plugin["beside_8_busy_streams_command"] = " ".join(os.path.relpath(c, ROOT) if os.path.isabs(c) else c for c in cmd)
            # what one batch costs the lane engine on its own (no plugin around it): eight 512 KiB requests per batch
            ebench = os.path.join(ROOT, "tests", "harness", "engine_bench")
            if os.path.exists(ebench):
                cmd = [ebench, flbuild.lib_path(), "--requests", "8", "--depth", "4", "--span-mib", "1024"]
                try:
                    res = subprocess.run(cmd, capture_output=True, text=True, timeout=120)
                    line = json.loads(res.stdout.strip().splitlines()[-1]) if res.returncode == 0 else None
                except Exception:
                    line = None
                if line and line.get("bit_exact"):
                    plugin["lane_engine_batch_of_8"] = {"one_at_a_time_us": line["one_at_a_time_us_per_batch"], "four_in_flight_us_per_batch": line["in_flight_us_per_batch"],
                                                        "four_in_flight_GBps_4N": line["in_flight_GBps_4N"], "buffers": "walking through 1 GiB", "bit_exact": True}
                else:
                    plugin["lane_engine_batch_of_8"] = None
                plugin["lane_engine_batch_of_8_command"] = " ".join(os.path.relpath(c, ROOT) if os.path.isabs(c) else c for c in cmd)

    import numpy as np
    import torch

    from fuselink_amd import core

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; there is no CPU fallback for the measured path", file=sys.stderr)
        return 3
    core.init(0)
    for kv in args.tune:
        key, _, val = kv.partition("=")
        core.tune(key, int(val))
    dev = torch.device("cuda:0")
    kind, nbytes, chunk, lanes, rows, epoch_len = WORKLOADS[args.workload]
    if args.lanes:
        lanes = args.lanes
    rng = np.random.default_rng(20251125)
    gen = torch.Generator(device=dev)
    gen.manual_seed(20251125)
    stream = torch.cuda.Stream(device=dev)
    status = core.new_status(dev)

    # ---- synthetic inputs, resident in HBM ------------------------------------------------------
    sizes_np = None
    if kind == "blocks":
        # cfg3 proper: 256 blocks of up to 4096 rows; more blocks mean finer dispatch, down to a token (one row) per block
        max_rows = 4096 if args.blocks == 256 else max(1, 65536 // args.blocks)
        ranks = np.arange(1, max_rows + 1, dtype=np.float64)
        p = ranks ** -1.1
        rows_per_block = rng.choice(np.arange(1, max_rows + 1), size=args.blocks, p=p / p.sum())
        sizes_np = (rows_per_block * 7168 * 2).astype(np.uint32)
        if args.ragged:
            sizes_np += rng.integers(1, 16, size=args.blocks).astype(np.uint32)
        nbytes = int(sizes_np.sum())
        credits_np = np.array([[4, 4, 4, 4, 4, 4, 4, 1]], dtype=np.int32)   # one lane at 25 % idleness
        n_chunks = args.blocks
    else:
        credits_np = rng.integers(1, 9, size=(rows, lanes)).astype(np.int32)
        n_chunks = (nbytes + chunk - 1) // chunk
    credits = torch.from_numpy(credits_np).to(dev)
    if args.workload.startswith("cfg2"):
        src = torch.randn(nbytes // 2, dtype=torch.float16, device=dev, generator=gen).view(torch.uint8)
    elif kind == "uniform":
        src = torch.randint(0, 2**31 - 1, (nbytes // 4,), dtype=torch.int32, device=dev, generator=gen).view(torch.uint8)
    else:
        src = torch.randint(-32768, 32767, ((nbytes + 1) // 2,), dtype=torch.int16, device=dev, generator=gen).view(torch.uint8)[:nbytes]
    dst = torch.zeros(nbytes, dtype=torch.uint8, device=dev)
    sizes = torch.from_numpy(sizes_np.view(np.int32)).to(dev) if sizes_np is not None else None
    page_bytes, ppc = 32768, 4
    tables = None
    if kind == "pages":
        half = nbytes // 2
        tables = [torch.from_numpy(rng.permutation(half // page_bytes).astype(np.int32)).to(dev) for _ in range(2)]

    # ---- registration-time work (untimed): table once for sizing, windows bound from the VMM pool --
    msg_bytes = nbytes // 2 if kind == "pages" else nbytes    # K and V are two messages over the same windows
    msg_chunks = n_chunks // 2 if kind == "pages" else n_chunks

    # a message too large for the Infinity Cache is striped in destination order (windows written front to back):
    # the scheduler then also emits the table's rows lane by lane
    # (measured: no gain for the paged gather, whose reads are scattered either way, so it keeps chunk order)
    by_lane = kind == "uniform" and rows <= 32 and nbytes > (256 << 20) and not args.no_by_lane

    use_tiles = kind == "blocks" and (args.tile_descriptors > 0 or
                                      (args.tile_descriptors < 0 and n_chunks >= 4096 and nbytes < 2 * core.TILE_BYTES * n_chunks))
    tiles_capacity = nbytes // core.TILE_BYTES + n_chunks if use_tiles else 0

    def run_schedule(out=None):
        return core.schedule(n_lanes=lanes, credits=credits, quantum=chunk, sizes=sizes,
                             total_bytes=0 if sizes is not None else msg_bytes, chunk_bytes=0 if sizes is not None else chunk,
                             epoch_len=epoch_len, out=out, stream=stream, by_lane=by_lane, tiles_capacity=tiles_capacity,
                             workspace=sizes is not None)   # a long variable list is then scanned by several workgroups

    sched = run_schedule()
    stream.synchronize()
    hdr = sched.hdr_numpy()
    lane_bytes = [int(b) for b in hdr["lane_bytes"][:lanes]]
    units = sum((b + core.UNIT_BYTES - 1) // core.UNIT_BYTES for b in lane_bytes)

    # ---- a fixed pool: the message goes in waves, every wave scheduled from the carried state with window offsets
    # from zero, and the windows are as large as the fullest wave needs (found here, untimed, from the headers) ----
    waves = None
    if args.pool_units > 0:
        if kind != "uniform" or (rows == 1 and epoch_len == 0 and args.path != "split"):
            print("bench.py: --pool-units applies to the table-driven uniform workloads (cfg5, or --path split)", file=sys.stderr)
            return 2
        state = core.new_state(dev)
        for k in range(1, 65):
            per = (n_chunks + k - 1) // k
            cuts = [(i * per * chunk, min(nbytes, (i + 1) * per * chunk)) for i in range(k) if i * per * chunk < nbytes]
            with torch.cuda.stream(stream):
                state.zero_()
            scheds, need = [], [0] * lanes
            for lo, hi in cuts:
                s_w = core.schedule(n_lanes=lanes, credits=credits, quantum=chunk, total_bytes=hi - lo, chunk_bytes=chunk, src_base=lo,
                                    epoch_len=epoch_len, mode=core.SCHED_RESET_OFFSETS, state=state, stream=stream, by_lane=by_lane)
                stream.synchronize()
                need = [max(a_, int(b_)) for a_, b_ in zip(need, s_w.hdr_numpy()["lane_bytes"][:lanes])]
                scheds.append(s_w)
            if sum((b_ + core.UNIT_BYTES - 1) // core.UNIT_BYTES for b_ in need) <= args.pool_units:
                waves = [(lo, hi, s_w, core.uniform_hint(hi - lo, chunk) if args.hint else None) for (lo, hi), s_w in zip(cuts, scheds)]
                lane_bytes = need
                units = sum((b_ + core.UNIT_BYTES - 1) // core.UNIT_BYTES for b_ in need)
                break
        if waves is None:
            print("bench.py: the message does not fit that pool in 64 waves", file=sys.stderr)
            return 2
    # ---- waves that keep the windows cache-resident: what one wave stages is read back by its own reassembly launch
    # before the next wave overwrites it, so the window traffic never reaches HBM ----
    cwaves = twaves = None
    wave_chunks = 0
    if (kind == "uniform" and not waves and args.cache_waves != 0 and args.path in ("auto", "fused") and nbytes > (256 << 20)
            and epoch_len > 0 and args.wave_epochs > 1 and args.wave_epochs * epoch_len * chunk <= (200 << 20)):
        # one scheduler launch whose rows restart their window offsets every wave, then a table-driven pair per wave
        wave_chunks = args.wave_epochs * epoch_len
        s_all = core.schedule(n_lanes=lanes, credits=credits, quantum=chunk, total_bytes=nbytes, chunk_bytes=chunk, epoch_len=epoch_len,
                              stream=stream, wave_chunks=wave_chunks)
        stream.synchronize()
        t_all = s_all.table_numpy()
        need = [0] * lanes
        twaves = []
        for w0 in range(0, n_chunks, wave_chunks):
            part = t_all[w0: w0 + wave_chunks]
            by = np.bincount(part["lane"], weights=part["len"].astype(np.float64), minlength=lanes)
            need = [max(a_, int(b_)) for a_, b_ in zip(need, by[:lanes])]
            lo, hi = w0 * chunk, min(nbytes, (w0 + wave_chunks) * chunk)
            twaves.append((w0, min(wave_chunks, n_chunks - w0), core.uniform_hint(hi - lo, chunk)))
        lane_bytes = need
        units = sum((b_ + core.UNIT_BYTES - 1) // core.UNIT_BYTES for b_ in need)
    elif (kind == "uniform" and not waves and args.cache_waves != 0 and args.path in ("auto", "fused") and nbytes > (256 << 20)
            and (rows == 1 or epoch_len > 0)):
        per = epoch_len * chunk if epoch_len else max(chunk, (64 << 20) // chunk * chunk)
        if per <= (96 << 20):
            cwaves, need = [], [0] * lanes
            for i, lo in enumerate(range(0, nbytes, per)):
                hi = min(nbytes, lo + per)
                row = credits_np[i % rows if epoch_len else 0].tolist()
                # with epochs every wave starts a new one; without, the quanta carry on from wave to wave
                u_w = core.uniform_params(hi - lo, chunk, row, src_base=lo, epoch_bytes=0 if epoch_len else lo)
                s_w = core.schedule(n_lanes=lanes, credits=row, quantum=chunk, total_bytes=hi - lo, chunk_bytes=chunk, stream=stream,
                                    state=None if epoch_len else _state_at(core, dev, lo, chunk), mode=core.SCHED_RESET_OFFSETS)
                stream.synchronize()
                need = [max(a_, int(b_)) for a_, b_ in zip(need, s_w.hdr_numpy()["lane_bytes"][:lanes])]
                cwaves.append(u_w)
            lane_bytes = need
            units = sum((b_ + core.UNIT_BYTES - 1) // core.UNIT_BYTES for b_ in need)
    pool = core.Pool(0, args.pool_units if waves else max(256, units))
    windows = []
    for b in lane_bytes:
        w = core.Window(pool, max(b, 1))
        w.bind(b)
        windows.append(w)
    win = core.make_windows([w.base for w in windows], [w.bound_bytes for w in windows])

    # header fields that follow from the uniform split alone; the kernels then need not wait for d_hdr
    hint = core.uniform_hint(msg_bytes, chunk) if (args.hint and kind == "uniform") else None
    carry = args.path == "carry"
    deliver = args.path == "deliver"
    if (carry or deliver) and (kind != "uniform" or rows != 1 or epoch_len != 0 or waves or cwaves or twaves):
        print("bench.py: --path carry and --path deliver take a uniform workload under one credit row that moves in one launch pair", file=sys.stderr)
        return 2
    fused = not waves and not cwaves and not twaves and kind in ("uniform", "pages") and (args.path in ("fused", "carry", "deliver") or (args.path == "auto" and rows == 1 and epoch_len == 0 and msg_chunks <= 65535))
    if fused and (rows != 1 or epoch_len != 0):
        print("bench.py: the fused path takes a single credit row without epochs", file=sys.stderr)
        return 2
    uni = core.uniform_params(msg_bytes, chunk, credits_np[0].tolist()) if fused else None
    landing_bufs = [torch.zeros(max(b, 1), dtype=torch.uint8, device=dev) for b in lane_bytes] if carry else None
    landing = core.make_windows([t.data_ptr() for t in landing_bufs], lane_bytes) if carry else None

    def step():
        if kind == "pages" and fused:
            for half_i in range(2):   # K, then V; the gather works each chunk's lane and offset out itself and writes the table
                lo = half_i * msg_bytes
                core.gather_pages_uniform(src[lo: lo + msg_bytes], tables[half_i], page_bytes, win, uni, status, out=sched, stream=stream)
                core.scatter_pages_uniform(dst[lo: lo + msg_bytes], tables[half_i], page_bytes, win, uni, status, stream=stream)
        elif kind == "pages":
            for half_i in range(2):   # K, then V: schedule, gather the pages into the windows, scatter them back out
                run_schedule(sched)
                lo = half_i * msg_bytes
                core.gather_pages(src[lo: lo + msg_bytes], tables[half_i], page_bytes, ppc, win, sched, status,
                                  use_lds=bool(args.lds), stream=stream, by_lane=by_lane)
                core.scatter_pages(dst[lo: lo + msg_bytes], tables[half_i], page_bytes, ppc, win, sched, status,
                                   use_lds=bool(args.lds), stream=stream)
        elif twaves:
            core.schedule(n_lanes=lanes, credits=credits, quantum=chunk, total_bytes=nbytes, chunk_bytes=chunk, epoch_len=epoch_len,
                          out=sched, stream=stream, wave_chunks=wave_chunks)
            for w0, cnt, h_w in twaves:
                sub = core.Schedule(sched.table[w0 * core.DESC_DTYPE.itemsize:], sched.hdr, cnt, core.TILE_BYTES)
                core.stripe(src, win, sub, status, stream=stream, hint=h_w)
                core.reassemble(dst, win, sub, status, stream=stream, hint=h_w)
        elif cwaves:
            for u_w in cwaves:
                core.stripe_uniform(src, win, u_w, status, out=sched, stream=stream)
                core.reassemble_uniform(dst, win, u_w, status, stream=stream)
        elif waves:
            with torch.cuda.stream(stream):
                state.zero_()
            for lo, hi, s_w, h_w in waves:
                core.schedule(n_lanes=lanes, credits=credits, quantum=chunk, total_bytes=hi - lo, chunk_bytes=chunk, src_base=lo, epoch_len=epoch_len,
                              mode=core.SCHED_RESET_OFFSETS, state=state, out=s_w, stream=stream, by_lane=by_lane)
                core.stripe(src, win, s_w, status, stream=stream, hint=h_w, by_lane=by_lane)
                core.reassemble(dst, win, s_w, status, stream=stream, hint=h_w)
        elif deliver:
            # staging and delivery in one launch (source -> staging windows and destination)
            core.stage_deliver_uniform(src, dst, win, uni, status, out=sched, stream=stream)
        elif carry:
            # staging and the wire in one launch (source -> staging windows -> landing windows), delivery out of the landing windows
            core.stripe_uniform_carry(src, win, landing, uni, status, out=sched, stream=stream)
            core.reassemble_uniform(dst, landing, uni, status, stream=stream)
        elif fused:
            # the striping launch computes each chunk's lane and offset itself and writes the table out
            core.stripe_uniform(src, win, uni, status, out=sched, stream=stream)
            core.reassemble_uniform(dst, win, uni, status, stream=stream)
        else:
            run_schedule(sched)
            core.stripe(src, win, sched, status, stream=stream, hint=hint, by_lane=by_lane)
            core.reassemble(dst, win, sched, status, stream=stream, hint=hint)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps

    # correctness of what was just timed: bit-exact round trip, no range refusals
    assert int(status.item()) == 0, "a kernel refused a chunk (window or buffer range)"
    assert torch.equal(src, dst), "reassembled buffer differs from the source"

    # ---- per-kernel durations: the same K steps again, every launch carrying its own start/stop HIP
    # events on the launch stream (they bracket the kernel alone; launches stay back to back) ----------
    def profiled(fn, launches):
        core.prof_begin(launches)
        fn()
        return core.prof_end(launches)

    def steps_again():
        for _ in range(args.steps):
            step()

    per = profiled(steps_again, (8 + 2 * len(cwaves or ()) + 3 * len(waves or ()) + 2 * len(twaves or ())) * args.steps)
    mean = lambda xs: sum(xs) / len(xs)
    out_k, in_k = ("gather", "scatter") if kind == "pages" else ("stage_deliver", "reassemble") if deliver else ("stripe", "reassemble")
    if deliver:
        per.setdefault(in_k, [0.0])   # (no second launch)
    stripe_us, reasm_us = mean(per[out_k]), mean(per[in_k])
    stripe_min, reasm_min = min(per[out_k]), min(per[in_k])
    launches_per_step = len(per[out_k]) // args.steps
    if fused or cwaves:
        # the table the fused launch wrote must be the scheduler kernel's table (with waves, sched holds the last wave's only)
        fused_table = sched.table_numpy().tobytes()

        def scheds():
            for _ in range(args.steps):
                run_schedule(sched)

        per_s = profiled(scheds, 2 * args.steps)
        assert cwaves or sched.table_numpy().tobytes() == fused_table, "fused and standalone scheduler tables differ"
        sched_us, n_sched = mean(per_s["schedule"]), len(per_s["schedule"]) // args.steps
    else:
        sched_us, n_sched = mean(per["schedule"]), len(per["schedule"]) // args.steps

    def copies():
        for _ in range(min(args.steps, 100)):
            core.copy(dst[:msg_bytes], src[:msg_bytes], stream=stream)

    copy_us = mean(profiled(copies, 128)["copy"])
    assert torch.equal(src, dst)

    def runtime_copy_us(d, s, reps):
        """The runtime's own device-to-device copy of the same bytes (hipMemcpyAsync, which torch's copy_ issues for
        contiguous bytes on one device): what a copy that stripes nothing gets from the vendor's path.  HIP events
        around every copy on the launch stream, back to back, mean -- as the library's per-launch timing does."""
        with torch.cuda.stream(stream):
            for _ in range(3):
                d.copy_(s)
            evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(reps)]
            for a, b in evs:
                a.record(stream)
                d.copy_(s)
                b.record(stream)
        stream.synchronize()
        return mean([a.elapsed_time(b) * 1e3 for a, b in evs])

    rt_copy_us = runtime_copy_us(dst[:msg_bytes], src[:msg_bytes], min(args.steps, 100))
    assert torch.equal(src, dst)

    # ---- the same step over rotating user buffers: the timed loop above re-reads one source and rewrites one
    # destination, which the 256 MB Infinity Cache partly holds from step to step; with enough pairs in rotation
    # (1 GiB of user buffers) every step meets them cold, as a stream of distinct messages would.  Reported
    # beside `value`, never as `value`.
    cold = None
    if args.cold_user_buffers and fused and kind == "uniform" and nbytes <= (128 << 20):
        cold_cmd = "python bench.py" + ("" if args.workload.startswith("cfg2") else f" --workload {args.workload}")
        pairs = max(2, (1 << 30) // (2 * nbytes))
        srcs = [src] + [torch.randint(0, 2**31 - 1, (nbytes // 4,), dtype=torch.int32, device=dev, generator=gen).view(torch.uint8)
                        for _ in range(pairs - 1)]
        dsts = [dst] + [torch.zeros(nbytes, dtype=torch.uint8, device=dev) for _ in range(pairs - 1)]

        def rotating_steps():
            for i in range(args.steps):
                core.stripe_uniform(srcs[i % pairs], win, uni, status, out=sched, stream=stream)
                core.reassemble_uniform(dsts[i % pairs], win, uni, status, stream=stream)

        rotating_steps()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        rotating_steps()
        torch.cuda.synchronize()
        cold_ms = (time.perf_counter() - t0) * 1e3 / args.steps
        per_c = profiled(rotating_steps, 4 * args.steps)
        assert int(status.item()) == 0
        assert all(torch.equal(a, b) for a, b in zip(srcs[: min(pairs, args.steps)], dsts)), "a rotating pair differs"
        cold = {"value": round(algo_bytes_cold(nbytes) / (cold_ms * 1e-3) / 1e9, 1), "unit": "GB/s", "ms_per_step": round(cold_ms, 5),
                "pairs": pairs, "user_buffer_bytes": 2 * pairs * nbytes,
                "kernels_us": {"stripe": round(mean(per_c["stripe"]), 2), "reassemble": round(mean(per_c["reassemble"]), 2)},
                "pct_of_hbm_peak": round(100.0 * algo_bytes_cold(nbytes) / (cold_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 2),
                "note": "same step, source/destination pairs in rotation so that no user buffer is cache-resident; windows reused",
                "command": cold_cmd}
        del srcs, dsts

    # ---- the same two kernels with HBM as the only server: one launch pair over 1 GiB in 64 KiB chunks on 16 lanes (the
    # stress configuration's shape under one credit row; 3 GiB of source, windows and destination, so nothing of one
    # launch is left in the 256 MB Infinity Cache for the next).  Goes into `roofline` beside the headline kernel's
    # fraction, which the cache helps.
    hbm_only = None
    if args.cold_user_buffers and fused and kind == "uniform" and nbytes <= (128 << 20):
        hb_n, hb_chunk, hb_lanes = 1 << 30, 64 << 10, 16
        hb_row = rng.integers(1, 9, size=hb_lanes).astype(np.int32).tolist()
        hb_src = torch.randint(0, 2**31 - 1, (hb_n // 4,), dtype=torch.int32, device=dev, generator=gen).view(torch.uint8)
        hb_dst = torch.zeros(hb_n, dtype=torch.uint8, device=dev)
        hb_s = core.schedule(n_lanes=hb_lanes, credits=hb_row, quantum=hb_chunk, total_bytes=hb_n, chunk_bytes=hb_chunk, stream=stream)
        stream.synchronize()
        hb_lane_bytes = [int(b) for b in hb_s.hdr_numpy()["lane_bytes"][:hb_lanes]]
        hb_pool = core.Pool(0, sum((b + core.UNIT_BYTES - 1) // core.UNIT_BYTES for b in hb_lane_bytes))
        hb_windows = []
        for b in hb_lane_bytes:
            w = core.Window(hb_pool, max(b, 1))
            w.bind(b)
            hb_windows.append(w)
        hb_win = core.make_windows([w.base for w in hb_windows], [w.bound_bytes for w in hb_windows])
        hb_uni = core.uniform_params(hb_n, hb_chunk, hb_row)
        hb_reps = 8

        def hb_pairs():
            for _ in range(hb_reps):
                core.stripe_uniform(hb_src, hb_win, hb_uni, status, stream=stream)
                core.reassemble_uniform(hb_dst, hb_win, hb_uni, status, stream=stream)

        def hb_copies():
            for _ in range(hb_reps):
                core.copy(hb_dst, hb_src, stream=stream)

        hb_pairs()
        per_h = profiled(hb_pairs, 4 * hb_reps)
        hb_copy_us = mean(profiled(hb_copies, 2 * hb_reps)["copy"])
        hb_rt_us = runtime_copy_us(hb_dst, hb_src, hb_reps)
        torch.cuda.synchronize()
        assert int(status.item()) == 0 and torch.equal(hb_src, hb_dst)
        hb_frac = lambda us: round(2 * hb_n / (us * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4)
        hbm_only = {"message_bytes": hb_n, "chunk_bytes": hb_chunk, "lanes": hb_lanes, "footprint_bytes": 3 * hb_n,
                    "stripe_us": round(mean(per_h["stripe"]), 1), "stripe_frac": hb_frac(mean(per_h["stripe"])),
                    "reassemble_us": round(mean(per_h["reassemble"]), 1), "reassemble_frac": hb_frac(mean(per_h["reassemble"])),
                    "plain_copy_us": round(hb_copy_us, 1), "plain_copy_frac": hb_frac(hb_copy_us),
                    "hipMemcpyAsync_us": round(hb_rt_us, 1), "hipMemcpyAsync_frac": hb_frac(hb_rt_us),
                    "timing": f"HIP events around every launch, mean of {hb_reps} launch pairs back to back, measured in this run",
                    "command": "python bench.py"}
        del hb_src, hb_dst
        for w in hb_windows:
            w.destroy()
        hb_pool.destroy()

    # ---- the scheduler kernels on a list long enough for a per-1000-chunk rate: the stress configuration's ----
    sched_bench = None
    if args.scheduler_bench:
        sb_n, sb_lanes, sb_rows, sb_epoch, sb_chunk = 16384, 16, 17, 1000, 64 << 10
        sb_credits = torch.from_numpy(rng.integers(1, 9, size=(sb_rows, sb_lanes)).astype(np.int32)).to(dev)
        sb_sizes_np = rng.integers(1, 2 * sb_chunk, size=sb_n).astype(np.uint32)      # variable sizes: the scan has to run
        sb_sizes = torch.from_numpy(sb_sizes_np.view(np.int32)).to(dev)
        reps = 50

        def sb_run(label, **kw):
            out_s = core.schedule(n_lanes=sb_lanes, credits=sb_credits, epoch_len=sb_epoch, stream=stream, **kw)   # buffers, untimed
            stream.synchronize()

            def go():
                for _ in range(reps):
                    core.schedule(n_lanes=sb_lanes, credits=sb_credits, epoch_len=sb_epoch, stream=stream, out=out_s, **kw)

            go()
            us = profiled(go, 4 * reps)["schedule"]
            launches = len(us) // reps
            per_call = sum(us) / reps
            return {"us_per_call": round(per_call, 2), "launches_per_call": launches, "us_per_1k_chunks": round(per_call / (sb_n / 1000.0), 3)}

        sched_bench = {
            "chunks": sb_n, "lanes": sb_lanes, "credit_rows": sb_rows, "epoch_len": sb_epoch,
            "closed_form_uniform_64KiB": sb_run("closed", quantum=sb_chunk, total_bytes=sb_n * sb_chunk, chunk_bytes=sb_chunk),
            "scan_variable_sizes_one_workgroup": sb_run("scan1", quantum=sb_chunk, sizes=sb_sizes),
            "scan_variable_sizes_workgroup_per_1024_chunks": sb_run("scanN", quantum=sb_chunk, sizes=sb_sizes, workspace=True),
            "timing": "HIP events around every scheduler launch, summed per call, mean of 50 calls back to back",
            "command": "python bench.py",
        }

    algo_bytes_step = 4 * nbytes          # stripe: read N + write N; reassemble: read N + write N
    algo_bytes_kernel = 2 * msg_bytes // len(waves or cwaves or twaves or (0,))    # one launch of the copy kernel (with waves: the average one)
    if deliver:
        algo_bytes_step = 3 * nbytes      # read N, write N into the windows, write N into the destination
    if carry or deliver:
        algo_bytes_kernel = 3 * msg_bytes   # read N, write N into the staging windows, write N into the landing windows (every vector loaded once, stored twice)
    value = algo_bytes_step / (ms_per_step * 1e-3) / 1e9
    pair_us = (stripe_us + reasm_us) * launches_per_step
    achieved = algo_bytes_kernel / (stripe_us * 1e-6) / 1e9
    if kind == "pages" and fused:
        kernel_name = "fl_copy_uniform_fused<0, FusedPageArgs> (gather)"
    elif kind == "pages":
        kernel_name = f"fl_page_tiles<0, lds={args.lds}> (gather)"
    elif deliver:
        kernel_name = "fl_copy_uniform_fused<0, FusedCarryArgs> (stage + deliver)"
    elif carry:
        kernel_name = "fl_copy_uniform_fused<0, FusedCarryArgs> (stripe + carry)"
    elif fused or cwaves:
        kernel_name = "fl_copy_uniform_fused<0> (stripe)"
    elif hint is not None:
        kernel_name = "fl_copy_uniform<0> (stripe)"
    elif use_tiles:
        kernel_name = "fl_copy_desc<0> (stripe)"
    else:
        kernel_name = "fl_copy_tiles<0> (stripe)"

    # which recorded counter measurement, if any, covers this run's dominant kernel on this workload
    if args.lanes or waves or twaves or (kind == "blocks" and args.blocks != 256):
        traffic_key = None
    elif cwaves:
        traffic_key = f"{args.workload}/{len(cwaves)} waves"
    elif carry or deliver:
        traffic_key = f"{args.workload}/{args.path}"
    else:
        traffic_key = args.workload
    out = {
        # the headline metric's own wording for the workload it is quoted on; `value` is its GB/s part, the percentage of the
        # HBM peak and the chunks per second travel as fields of their own (pct_of_hbm_peak, chunks_per_s)
        "metric": ("stripe+reassemble GB/s (% of 8 TB/s HBM) + chunks/s, 64 MiB over 8 lanes" if args.workload.startswith("cfg2")
                   else "stripe+reassemble GB/s (% of 8 TB/s HBM) + chunks/s"),
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u8",
        "data": "synthetic",
        "config": {"workload": args.workload, "bytes": nbytes, "chunk_bytes": chunk if sizes is None else "variable", "chunks": n_chunks,
                   "lanes": lanes, "credits": credits_np.tolist() if rows == 1 else f"{rows} seeded rows in [1,8]", "epoch_len": epoch_len,
                   "step": ("2x(gather(with scheduler folded in)+scatter)" if (kind == "pages" and fused) else "2x(schedule+gather+scatter)" if kind == "pages" else
                            "stripe(with scheduler folded in)+carry into landing windows, then reassemble out of them" if carry else
                            "one launch: stage into the windows (scheduler folded in) and deliver into the destination; value counts 3 x bytes" if deliver else
                            "stripe(with scheduler folded in)+reassemble" if fused else
                            f"{len(cwaves)} waves of stripe(with scheduler folded in)+reassemble over cache-resident windows" if cwaves else
                            f"schedule, then {len(twaves)} waves of stripe+reassemble over cache-resident windows" if twaves else "schedule+stripe+reassemble"),
                   "launch": "eager", "windows": f"HIP VMM, {units} units of 2 MiB bound" + (f", pool of {args.pool_units}, {len(waves)} waves" if waves else ""), "tile_descriptors": bool(use_tiles),
                   "stripe_order": "chunk" if (cwaves or twaves) else "destination (lane by lane)" if (by_lane and not fused) else "chunk (destination order inside the kernel for messages past 256 MiB)" if fused else "chunk"},
        "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBPS, 2),
        "chunks_per_s": round(n_chunks / (ms_per_step * 1e-3), 1),
        "kernels_us": {"schedule": round(sched_us, 2), out_k: round(stripe_us, 2), in_k: round(reasm_us, 2),
                       out_k + "_min": round(stripe_min, 2), in_k + "_min": round(reasm_min, 2),
                       "plain_copy_same_bytes": round(copy_us, 2), "hipMemcpyAsync_same_bytes": round(rt_copy_us, 2)},
        "stripe_reassemble_pair_GBps": round(algo_bytes_step / (pair_us * 1e-6) / 1e9, 1),
        "scheduler_kernel": "standalone launch, not part of the fused step" if (fused or cwaves) else "first launch of every message",
        # one launch schedules a whole message; below 1000 chunks its cost is the flat launch time, not a per-1k rate
        "scheduler_launch_us": round(sched_us, 2),
        # the rate on a list long enough to have one: the stress configuration's 16384 chunks through the prefix-scan kernels
        # (a workgroup per 1024 chunks); the other scheduler shapes are in scheduler_bench
        "scheduler_us_per_1k_chunks": (sched_bench["scan_variable_sizes_workgroup_per_1024_chunks"]["us_per_1k_chunks"] if sched_bench else
                                       round(sched_us * n_sched / (n_chunks / 1000.0), 3) if n_chunks >= 1000 else None),
        "scheduler_bench": sched_bench,
        "cold_user_buffers": cold,
        "plugin_abi": plugin,
        "roofline": {"bound": "hbm", "kernel": kernel_name, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     # what the fraction means for this workload: cached footprints are served in part by the 256 MB Infinity Cache
                     "note": ("footprint (source, windows, destination) of %d MiB: %s" % (
                         3 * nbytes >> 20, "largely resident in the 256 MB Infinity Cache, so this is a fraction of the HBM peak reached with that cache's help; "
                         "the same kernels with HBM as the only server are in hbm_only (measured in this run; as a whole workload: bench.py --workload cfg5_stress_1GiB_64KiB_16lanes --cache-waves 0)"
                         if 3 * nbytes <= (256 << 20) else "beyond the 256 MB Infinity Cache" + (
                             "; moved in cache-resident waves, the windows' traffic stays in the cache" if cwaves else ": every byte is served by HBM"))) if kind == "uniform" else None,
                     "traffic": MEASURED_TRAFFIC.get(traffic_key) if traffic_key else None},
    }
    if out["roofline"]["traffic"] is not None:
        # a recorded measurement (two rocprofv3 --pmc runs, scaled by a plain copy of known size), not read in this run
        out["roofline"]["traffic_source"] = TRAFFIC_SOURCE.get(traffic_key)
    if hbm_only is not None:
        out["roofline"]["hbm_only"] = hbm_only

    # ---- CPU baseline: the oracle's host-memcpy striping on a bounded sample ------------------------
    if not args.no_cpu_baseline:
        from tests import oracle_binding as ob
        src_np = src.cpu().numpy()
        cores = ob.lib().fl_cpu_cores()
        thr = min(lanes, cores, 16)
        if kind == "pages":
            tab, h, _ = ob.credit_schedule(n_lanes=lanes, credits=credits_np, quantum=chunk, total_bytes=msg_bytes, chunk_bytes=chunk)
            caps = h["lane_bytes"][:lanes]
            ts = []
            for _ in range(max(3, args.cpu_iters // 100)):
                c0 = time.perf_counter()
                for half_i in range(2):
                    half = src_np[half_i * msg_bytes: (half_i + 1) * msg_bytes]
                    tb = tables[half_i].cpu().numpy().view(np.uint32)
                    w_ = ob.cpu_gather_pages(half, tb, page_bytes, ppc, tab, caps)
                    back = ob.cpu_scatter_pages(msg_bytes, tb, page_bytes, ppc, w_, tab)
                ts.append(time.perf_counter() - c0)
                assert (back == half).all()
            med1 = sorted(ts)[len(ts) // 2]
            out["cpu_baseline"] = {"value": round(algo_bytes_step / med1 / 1e9, 2), "unit": "GB/s", "cores": 1, "kind": "port",
                                   "sample": f"{len(ts)} passes of the same K+V gather/scatter (host memcpy per page; includes "
                                             f"allocating the host windows each pass), median; host has {cores} cores"}
        else:
            tab, h, _ = ob.credit_schedule(n_lanes=lanes, credits=credits_np, quantum=chunk, sizes=sizes_np,
                                           total_bytes=0 if sizes_np is not None else nbytes,
                                           chunk_bytes=0 if sizes_np is not None else chunk, epoch_len=epoch_len)
            iters = args.cpu_iters if nbytes <= (64 << 20) else max(3, args.cpu_iters * (64 << 20) // nbytes)
            med1, _ = ob.cpu_baseline(src_np, tab, h, lanes, threads=1, warm=3, iters=iters)
            medm, _ = ob.cpu_baseline(src_np, tab, h, lanes, threads=thr, warm=3, iters=iters)
            out["cpu_baseline"] = {"value": round(algo_bytes_step / med1 / 1e9, 2), "unit": "GB/s", "cores": 1, "kind": "port",
                                   "sample": f"{iters} timed stripe+reassemble passes of the same {nbytes >> 20} MiB message "
                                             f"(host memcpy per chunk into 2 MiB-aligned lane windows), median; host has {cores} cores"}
            out["cpu_baseline_per_lane_threads"] = {"value": round(algo_bytes_step / medm / 1e9, 2), "unit": "GB/s", "cores": thr,
                                                    "kind": "port", "sample": "same passes, one pinned thread per lane"}
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
