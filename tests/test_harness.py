"""The C++ plugin harness (two proxy threads, dlopen + dlsym like a communication library)."""
import json
import os
import subprocess

import pytest

from fuselink_amd import build

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "harness", "plugin_harness")


def _run(args, env=None):
    if not os.path.exists(BIN):
        build.build_harness(verbose=False)
    e = dict(os.environ)
    e.update(env or {})
    res = subprocess.run([BIN, build.lib_path(), *args], capture_output=True, text=True, timeout=300, env=e)
    assert res.returncode == 0, res.stderr[-2000:]
    lines = [json.loads(l) for l in res.stdout.strip().splitlines() if l.startswith("{")]
    out = lines[-1]
    if len(lines) > 1:
        out["handoff"] = lines[-2]
    return out


@pytest.mark.parametrize("version", [6, 7, 8])
def test_harness_host_memory_two_threads(version):
    out = _run(["--host", "--bytes", str(16 << 20), "--request", str(1 << 20), "--inflight", "4", "--iters", "2",
                "--version", str(version)])
    assert out["bit_exact"] and out["requests"] == 16 and out["name"] == "FuseLink"


def test_harness_cfg1_host_reference_operating_point():
    # 4 MiB uint8 message, 512 KiB requests (one NCCL step each), as the reference's experiment drives the plugin
    out = _run(["--host", "--bytes", str(4 << 20), "--request", str(512 << 10), "--inflight", "8", "--iters", "3"],
               env={"NCCL_FUSELINK_LANES": "2", "NCCL_FUSELINK_CREDITS": "1,1"})
    assert out["bit_exact"] and out["requests"] == 8 and out["devices"] == 2


@pytest.mark.gpu
def test_harness_device_memory_cfg2_shape():
    out = _run(["--bytes", str(64 << 20), "--request", str(64 << 20), "--inflight", "1", "--iters", "5"],
               env={"NCCL_FUSELINK_LANES": "8", "NCCL_FUSELINK_CHUNKSIZE": str(256 << 10), "NCCL_FUSELINK_WINDOW_UNITS": "28",
                    "NCCL_FUSELINK_CREDITS": "8,6,7,1,8,7,3,3"})
    assert out["bit_exact"] and out["memory"] == "device"
    print(out)


@pytest.mark.gpu
def test_harness_device_memory_stress_four_in_flight():
    out = _run(["--bytes", str(1 << 30), "--request", str(64 << 20), "--inflight", "4", "--iters", "2"],
               env={"NCCL_FUSELINK_LANES": "16", "NCCL_FUSELINK_CHUNKSIZE": str(64 << 10), "NCCL_FUSELINK_WINDOW_UNITS": "4"})
    assert out["bit_exact"] and out["requests"] == 16
    print(out)


def test_harness_host_four_concurrent_connections():
    out = _run(["--host", "--bytes", str(8 << 20), "--request", str(1 << 20), "--inflight", "4", "--iters", "3", "--connections", "4"])
    assert out["bit_exact"] and out["connections"] == 4


@pytest.mark.gpu
def test_harness_device_four_concurrent_connections():
    # four connections stage through the same unit pool and monitor table at once, each on its own stream
    out = _run(["--bytes", str(128 << 20), "--request", str(16 << 20), "--inflight", "4", "--iters", "3", "--connections", "4"],
               env={"NCCL_FUSELINK_LANES": "8", "NCCL_FUSELINK_CHUNKSIZE": str(256 << 10)})
    assert out["bit_exact"] and out["connections"] == 4
    print(out)


def test_harness_kv_handoff_group_host_memory():
    # the five sends of the serving experiment's prefill -> decode hand-off (experiments/serving/model.hh:286-309):
    # int64 context output, K cache, V cache, int64 block table, int64 block counts; tiny and large messages mixed
    out = _run(["--host", "--handoff", "4,8,2,8,16,128", "--request", str(512 << 10), "--inflight", "8", "--iters", "2"])
    h = out["handoff"]
    assert out["bit_exact"] and h["cache_bytes_each"] == 2 * 32 * 2 * 8 * 16 * 128
    assert h["comm_volume_bytes"] == 2 * h["cache_bytes_each"] + 8 * 4 + 8 * 32 + 8 * 4
    assert out["requests"] == 1 + 4 + 4 + 1 + 1


@pytest.mark.gpu
def test_harness_kv_handoff_group_device_memory():
    # 8 requests x 64 blocks, 4 layers, 8 KV heads, 16-token blocks, head_dim 128, fp16: 64 MiB each for K and V,
    # cut into 512 KiB requests (NCCL_P2P_NET_CHUNKSIZE of the experiment), 8 in flight (NCCL_STEPS)
    out = _run(["--handoff", "8,64,4,8,16,128", "--request", str(512 << 10), "--inflight", "8", "--iters", "3"],
               env={"NCCL_FUSELINK_LANES": "8", "NCCL_FUSELINK_CHUNKSIZE": str(64 << 10)})
    assert out["bit_exact"] and out["handoff"]["cache_bytes_each"] == 64 << 20
    print(out["handoff"])


def test_plugin_host_path_under_thread_sanitizer():
    """Four connections, eight proxy threads, host memory: the plugin's request tables, FIFO, registry,
    credit row and monitor table are touched from all of them; ThreadSanitizer must stay silent."""
    lib, exe = build.build_tsan(verbose=False)
    env = dict(os.environ, TSAN_OPTIONS="halt_on_error=1 exitcode=66")
    res = subprocess.run([exe, lib, "--host", "--bytes", str(4 << 20), "--request", str(256 << 10), "--connections", "4",
                          "--inflight", "4", "--iters", "2"], capture_output=True, text=True, timeout=600, env=env)
    assert "ThreadSanitizer" not in res.stderr, res.stderr[-3000:]
    assert res.returncode == 0, res.stderr[-2000:]
    assert json.loads(res.stdout.strip().splitlines()[-1])["bit_exact"]


def test_plugin_host_path_under_address_sanitizer():
    """The same traffic with AddressSanitizer on the host code (leak check included): connections, requests,
    memory handles and listen comms are created and released many times over."""
    lib, exe = build.build_tsan(verbose=False, sanitizer="address")
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:exitcode=67:protect_shadow_gap=0")
    res = subprocess.run([exe, lib, "--host", "--bytes", str(4 << 20), "--request", str(256 << 10), "--connections", "4",
                          "--inflight", "4", "--iters", "3"], capture_output=True, text=True, timeout=600, env=env)
    assert "AddressSanitizer" not in res.stderr and "LeakSanitizer" not in res.stderr, res.stderr[-3000:]
    assert res.returncode == 0, res.stderr[-2000:]
    assert json.loads(res.stdout.strip().splitlines()[-1])["bit_exact"]


@pytest.mark.gpu
def test_the_resident_engine_does_not_hold_a_hardware_queue_for_as_long_as_requests_come():
    """A process has fewer hardware queues than an application has streams; the runtime puts several streams on one queue,
    and a kernel that never ends holds its queue.  With eight more streams of the process busy with small fills beside a
    connection at NCCL's request shape (about 5 ms of uninterrupted small requests per iteration), no fill may wait for
    the whole of that: the lane engine leaves after NCCL_FUSELINK_ENGINE_RESIDENT_US (1000) and is started again."""
    if not os.path.exists(BIN):
        build.build_harness(verbose=False)
    res = subprocess.run([BIN, build.lib_path(), "--bytes", str(1 << 30), "--request", str(512 << 10), "--inflight", "8", "--iters", "3", "--side-streams", "8"],
                         capture_output=True, text=True, timeout=300,
                         env=dict(os.environ, NCCL_FUSELINK_LANES="8", NCCL_FUSELINK_CHUNKSIZE=str(256 << 10)))
    assert res.returncode == 0, res.stderr[-2000:]
    lines = {l["harness"]: l for l in (json.loads(x) for x in res.stdout.strip().splitlines() if x.startswith("{"))}
    assert lines["plugin"]["bit_exact"] and lines["side_streams"]["streams"] == 8 and lines["side_streams"]["fills"] > 100
    print(lines["side_streams"], lines["plugin"]["GBps_4N_best"])
    assert lines["side_streams"]["fill_us_max"] < 3000, lines["side_streams"]


# ---- sender and receiver in two processes ----------------------------------------------------------------------------
# The receiver is a child forked before either side has loaded the plugin or touched the GPU; the two meet through the
# 128-byte handle alone (a POSIX shared-memory object named in it carries the descriptor ring; a second one, per pair of
# processes, the wave completions; the receiver's memory is opened by the sender through HIP IPC).  The child compares
# what it received with the pattern of the iteration and reports through its exit status.  Every shape runs both ways a
# wave can travel: written by the sender into the posted buffers through their registrations (NCCL_FUSELINK_WIRE_DIRECT=1,
# the default) and through the landing windows, delivered by the receiver's own engine or launches (0).
DIRECT = pytest.mark.parametrize("direct", [1, 0])


@pytest.mark.gpu
@DIRECT
def test_two_processes_cfg1_shape(direct):
    # the reference's own experiment: 4 MiB in 512 KiB chunks over 2 lanes, one request per NCCL step
    out = _run(["--two-process", "--bytes", str(4 << 20), "--request", str(512 << 10), "--inflight", "8", "--iters", "3"],
               env={"NCCL_FUSELINK_LANES": "2", "NCCL_FUSELINK_CHUNKSIZE": str(512 << 10), "NCCL_FUSELINK_CREDITS": "1,1", "NCCL_FUSELINK_WIRE_DIRECT": str(direct)})
    assert out["harness"] == "plugin_two_process" and out["bit_exact"] and out["requests"] == 8
    print(out)


@pytest.mark.gpu
@DIRECT
def test_two_processes_cfg2_shape(direct):
    # 64 MiB in 256 KiB chunks over 8 lanes with uneven credits, one request; the windows hold the message in one wave
    out = _run(["--two-process", "--bytes", str(64 << 20), "--request", str(64 << 20), "--inflight", "1", "--iters", "3"],
               env={"NCCL_FUSELINK_LANES": "8", "NCCL_FUSELINK_CHUNKSIZE": str(256 << 10), "NCCL_FUSELINK_WINDOW_UNITS": "28",
                    "NCCL_FUSELINK_CREDITS": "8,6,7,1,8,7,3,3", "NCCL_FUSELINK_WIRE_DIRECT": str(direct)})
    assert out["harness"] == "plugin_two_process" and out["bit_exact"] and out["requests"] == 1
    print(out)


@pytest.mark.gpu
@pytest.mark.parametrize("sets,direct", [(1, 0), (2, 0), (5, 0), (2, 1)])
def test_two_processes_requests_larger_than_the_windows_and_a_ragged_tail(sets, direct):
    # every request takes several waves through the landing windows (4 units per lane; `sets` sets of them, so that many
    # waves are on the wire at once), the last request is short and odd
    out = _run(["--two-process", "--bytes", str((96 << 20) + 12345), "--request", str(32 << 20), "--inflight", "2", "--iters", "2"],
               env={"NCCL_FUSELINK_LANES": "4", "NCCL_FUSELINK_CHUNKSIZE": str(128 << 10), "NCCL_FUSELINK_WINDOW_UNITS": "4",
                    "NCCL_FUSELINK_CREDITS": "3,1,2,2", "NCCL_FUSELINK_WIRE_SETS": str(sets), "NCCL_FUSELINK_WIRE_DIRECT": str(direct)})
    assert out["bit_exact"] and out["requests"] == 4
    print(out)


@pytest.mark.gpu
@DIRECT
def test_two_processes_many_small_requests_in_flight(direct):
    # NCCL's request shape across the process boundary: 512 KiB requests, 8 in flight, more requests than the descriptor
    # ring and the wave ring have slots (both wrap)
    out = _run(["--two-process", "--bytes", str(192 << 20), "--request", str(512 << 10), "--inflight", "8", "--iters", "2"],
               env={"NCCL_FUSELINK_LANES": "8", "NCCL_FUSELINK_CHUNKSIZE": str(256 << 10), "NCCL_FUSELINK_WIRE_SETS": "4", "NCCL_FUSELINK_WIRE_DIRECT": str(direct)})
    assert out["bit_exact"] and out["requests"] == 384
    print(out)


@pytest.mark.gpu
@DIRECT
def test_two_processes_kv_handoff_group(direct):
    # the prefill -> decode hand-off of the serving experiment (experiments/serving/model.hh:286-309), where the two are
    # different processes: five messages (int64 context output, K cache, V cache, int64 block table, int64 counts), each
    # a buffer and a registration of its own on either side, tiny and large mixed, cut into 512 KiB requests
    out = _run(["--two-process", "--handoff", "4,8,2,8,16,128", "--request", str(512 << 10), "--inflight", "8", "--iters", "2"], env={"NCCL_FUSELINK_WIRE_DIRECT": str(direct)})
    cache = 2 * 32 * 2 * 8 * 16 * 128
    assert out["bit_exact"] and out["group"] == "kv_handoff" and out["messages"] == 5
    assert out["bytes"] == 2 * cache + 8 * 4 + 8 * 32 + 8 * 4 and out["requests"] == 1 + 4 + 4 + 1 + 1
    print(out)
