"""Plugin test harness: loads libnccl-net-fuselink.so the way a communication library does
(dlopen + dlsym of the `ncclNetPlugin_v*` data symbol) and drives the function table.

Method names and argument meaning follow the table of the reference (FuseLink
src/extern/nccl_net.h:41-94): init / devices / getProperties / listen / connect / accept / regMr /
deregMr / isend / irecv / iflush / test / closeSend / closeRecv / closeListen.  Every method returns
the raw ncclResult_t first, so tests can assert on the error convention ("would block" is
ncclSuccess with a NULL comm or request)."""
from __future__ import annotations

import ctypes as C
import os
from typing import List, Optional, Tuple

from .build import lib_path

ncclSuccess, ncclUnhandledCudaError, ncclSystemError, ncclInternalError = 0, 1, 2, 3
ncclInvalidArgument, ncclInvalidUsage, ncclRemoteError, ncclInProgress = 4, 5, 6, 7
NCCL_PTR_HOST, NCCL_PTR_CUDA, NCCL_PTR_DMABUF = 1, 2, 4
NCCL_NET_HANDLE_MAXSIZE = 128

LOGGER = C.CFUNCTYPE(None, C.c_int, C.c_ulong, C.c_char_p, C.c_int, C.c_char_p)
R = C.c_int
VP = C.c_void_p
PVP = C.POINTER(C.c_void_p)
PI = C.POINTER(C.c_int)


class PropsV6(C.Structure):
    _fields_ = [("name", C.c_char_p), ("pciPath", C.c_char_p), ("guid", C.c_uint64), ("ptrSupport", C.c_int),
                ("speed", C.c_int), ("port", C.c_int), ("latency", C.c_float), ("maxComms", C.c_int), ("maxRecvs", C.c_int)]


class PropsV7(C.Structure):
    _fields_ = PropsV6._fields_ + [("netDeviceType", C.c_int), ("netDeviceVersion", C.c_int)]


class PropsV8(C.Structure):
    _fields_ = [("name", C.c_char_p), ("pciPath", C.c_char_p), ("guid", C.c_uint64), ("ptrSupport", C.c_int),
                ("regIsGlobal", C.c_int), ("speed", C.c_int), ("port", C.c_int), ("latency", C.c_float),
                ("maxComms", C.c_int), ("maxRecvs", C.c_int), ("netDeviceType", C.c_int), ("netDeviceVersion", C.c_int)]


def _table(version: int):
    props = {6: PropsV6, 7: PropsV7, 8: PropsV8}[version]
    size_t = C.c_size_t if version >= 8 else C.c_int
    conn = [C.c_int, VP, PVP] + ([PVP] if version >= 7 else [])
    acc = [VP, PVP] + ([PVP] if version >= 7 else [])
    fields = [
        ("name", C.c_char_p),
        ("init", C.CFUNCTYPE(R, LOGGER)),
        ("devices", C.CFUNCTYPE(R, PI)),
        ("getProperties", C.CFUNCTYPE(R, C.c_int, C.POINTER(props))),
        ("listen", C.CFUNCTYPE(R, C.c_int, VP, PVP)),
        ("connect", C.CFUNCTYPE(R, *conn)),
        ("accept", C.CFUNCTYPE(R, *acc)),
        ("regMr", C.CFUNCTYPE(R, VP, VP, size_t, C.c_int, PVP)),
        ("regMrDmaBuf", C.CFUNCTYPE(R, VP, VP, C.c_size_t, C.c_int, C.c_uint64, C.c_int, PVP)),
        ("deregMr", C.CFUNCTYPE(R, VP, VP)),
        ("isend", C.CFUNCTYPE(R, VP, VP, C.c_int, C.c_int, VP, PVP)),
        ("irecv", C.CFUNCTYPE(R, VP, C.c_int, PVP, PI, PI, PVP, PVP)),
        ("iflush", C.CFUNCTYPE(R, VP, C.c_int, PVP, PI, PVP, PVP)),
        ("test", C.CFUNCTYPE(R, VP, PI, PI)),
        ("closeSend", C.CFUNCTYPE(R, VP)),
        ("closeRecv", C.CFUNCTYPE(R, VP)),
        ("closeListen", C.CFUNCTYPE(R, VP)),
    ]
    if version >= 7:
        fields += [("getDeviceMr", VP), ("irecvConsumed", VP)]
    return type(f"NcclNetV{version}", (C.Structure,), {"_fields_": fields}), props


PLUGIN_SYMBOLS = ["ncclNetPlugin_v8", "ncclNetPlugin_v7", "ncclNetPlugin_v6"]
CONTROL_SYMBOLS = ["fl_monitor_attach_shm", "fl_monitor_detach", "fl_monitor_is_shared", "fl_monitor_daemon_running", "fl_monitor_reset", "fl_monitor_set_entry", "fl_monitor_set_clock", "fl_monitor_now", "fl_monitor_mark_active", "fl_monitor_tick",
                   "fl_monitor_status", "fl_monitor_idle_pick", "fl_monitor_release", "fl_monitor_credits", "fl_monitor_tx_mask", "fl_monitor_rx_credits", "fl_net_set_credits",
                   "fl_net_inject_fault", "fl_net_comm_stats", "fl_net_mask_stats", "fl_net_free_requests", "fl_net_launch_stats", "fl_net_last_table", "fl_net_last_launch",
                   "fl_net_flush", "fl_net_host_stats", "fl_net_timeline", "fl_net_reset"]


class LaunchSeg(C.Structure):
    _fields_ = [("channel", C.c_int32), ("first_row", C.c_uint32), ("n_rows", C.c_uint32), ("n_req", C.c_uint32),
                ("epoch_bytes", C.c_uint64), ("lane_base", C.c_uint64 * 16)]


class NetPlugin:
    """One loaded plugin table.  `version` picks ncclNetPlugin_v8 / _v7 / _v6."""

    def __init__(self, version: int = 8, path: Optional[str] = None, log: bool = False):
        path = path or os.environ.get("FUSELINK_LIB", lib_path())
        if not os.path.exists(path):
            raise ImportError(f"{path} is missing: build it with `python -m fuselink_amd.build`")
        self.lib = C.CDLL(path, mode=C.RTLD_GLOBAL)
        self.version = version
        table_t, self.props_t = _table(version)
        self.t = table_t.in_dll(self.lib, f"ncclNetPlugin_v{version}")
        self.messages: List[Tuple[int, str]] = []

        def _logger(level, flags, file, line, fmt):
            # the format arguments are not forwarded through ctypes; the format string names the event
            self.messages.append((level, (fmt or b"").decode(errors="replace")))
            if log:
                print(f"[plugin log {level}] {(fmt or b'').decode(errors='replace')}")

        self._logger = LOGGER(_logger)
        L = self.lib
        L.fl_monitor_reset.restype = C.c_int
        L.fl_monitor_attach_shm.argtypes = [C.c_char_p, C.c_char_p, C.c_int]
        L.fl_monitor_set_clock.argtypes = [C.c_int, C.c_int64]
        L.fl_monitor_now.restype = C.c_int64
        L.fl_monitor_mark_active.argtypes = [C.c_int, C.c_int, C.c_int64]
        L.fl_monitor_tick.argtypes = [C.c_int64]
        L.fl_monitor_set_entry.argtypes = [C.c_int, C.c_int, C.c_int32, C.c_int64]
        L.fl_monitor_status.argtypes = [C.c_int, C.c_int, C.POINTER(C.c_int32)]
        L.fl_monitor_idle_pick.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int]
        L.fl_monitor_credits.argtypes = [C.c_int, C.c_int, C.c_uint32, C.POINTER(C.c_uint32)]
        L.fl_net_set_credits.argtypes = [C.POINTER(C.c_uint32), C.c_int]
        L.fl_net_inject_fault.argtypes = [VP]
        L.fl_net_comm_stats.argtypes = [VP, C.POINTER(C.c_int64), C.POINTER(C.c_int64), C.POINTER(C.c_int64)]
        L.fl_net_launch_stats.argtypes = [VP, C.POINTER(C.c_int64), C.POINTER(C.c_int64)]
        L.fl_net_mask_stats.argtypes = [VP, C.POINTER(C.c_uint32), C.POINTER(C.c_int64)]
        L.fl_net_free_requests.argtypes = [VP]
        L.fl_monitor_tx_mask.argtypes = [C.c_int, C.c_int, C.POINTER(C.c_uint32)]
        L.fl_monitor_rx_credits.argtypes = [C.c_int, C.c_int, C.c_uint32, C.c_uint32, C.POINTER(C.c_uint32)]
        L.fl_net_last_table.argtypes = [VP, VP, C.c_int, VP]
        L.fl_net_last_launch.argtypes = [VP, C.POINTER(LaunchSeg), C.c_int, VP, C.c_int, VP]
        L.fl_net_flush.argtypes = [VP]

    # ---- the function table -----------------------------------------------------------------------
    @property
    def name(self) -> str:
        return self.t.name.decode()

    def init(self) -> int:
        return self.t.init(self._logger)

    def devices(self) -> Tuple[int, int]:
        n = C.c_int(-1)
        return self.t.devices(C.byref(n)), n.value

    def getProperties(self, dev: int):
        p = self.props_t()
        return self.t.getProperties(dev, C.byref(p)), p

    def listen(self, dev: int):
        handle = C.create_string_buffer(NCCL_NET_HANDLE_MAXSIZE)
        comm = C.c_void_p()
        rc = self.t.listen(dev, C.cast(handle, VP), C.byref(comm))
        return rc, handle, comm.value

    def connect(self, dev: int, handle):
        comm = C.c_void_p()
        if self.version >= 7:
            rc = self.t.connect(dev, C.cast(handle, VP), C.byref(comm), None)
        else:
            rc = self.t.connect(dev, C.cast(handle, VP), C.byref(comm))
        return rc, comm.value

    def accept(self, listen_comm):
        comm = C.c_void_p()
        if self.version >= 7:
            rc = self.t.accept(listen_comm, C.byref(comm), None)
        else:
            rc = self.t.accept(listen_comm, C.byref(comm))
        return rc, comm.value

    def regMr(self, comm, data: int, size: int, ptr_type: int):
        mh = C.c_void_p()
        rc = self.t.regMr(comm, C.c_void_p(data), size, ptr_type, C.byref(mh))
        return rc, mh.value

    def regMrDmaBuf(self, comm, data: int, size: int, ptr_type: int, offset: int = 0, fd: int = -1):
        mh = C.c_void_p()
        rc = self.t.regMrDmaBuf(comm, C.c_void_p(data), size, ptr_type, offset, fd, C.byref(mh))
        return rc, mh.value

    def regMrDmaBuf(self, comm, data: int, size: int, ptr_type: int, offset: int, fd: int):
        mh = C.c_void_p()
        rc = self.t.regMrDmaBuf(comm, C.c_void_p(data), size, ptr_type, offset, fd, C.byref(mh))
        return rc, mh.value

    def deregMr(self, comm, mhandle) -> int:
        return self.t.deregMr(comm, mhandle)

    def isend(self, send_comm, data: int, size: int, tag: int, mhandle):
        req = C.c_void_p()
        rc = self.t.isend(send_comm, C.c_void_p(data), size, tag, mhandle, C.byref(req))
        return rc, req.value

    def irecv(self, recv_comm, datas: List[int], sizes: List[int], tags: List[int], mhandles: List[int]):
        n = len(datas)
        d = (C.c_void_p * n)(*datas)
        s = (C.c_int * n)(*sizes)
        t = (C.c_int * n)(*tags)
        m = (C.c_void_p * n)(*mhandles)
        req = C.c_void_p()
        rc = self.t.irecv(recv_comm, n, d, s, t, m, C.byref(req))
        return rc, req.value

    def iflush(self, recv_comm, datas: List[int], sizes: List[int], mhandles: List[int]):
        n = len(datas)
        d = (C.c_void_p * n)(*datas)
        s = (C.c_int * n)(*sizes)
        m = (C.c_void_p * n)(*mhandles)
        req = C.c_void_p()
        rc = self.t.iflush(recv_comm, n, d, s, m, C.byref(req))
        return rc, req.value

    def test(self, request):
        done = C.c_int(0)
        size = C.c_int(-1)
        rc = self.t.test(request, C.byref(done), C.byref(size))
        return rc, done.value, size.value

    def closeSend(self, comm) -> int:
        return self.t.closeSend(comm)

    def closeRecv(self, comm) -> int:
        return self.t.closeRecv(comm)

    def closeListen(self, comm) -> int:
        return self.t.closeListen(comm)

    # ---- what NCCL's proxy does around the table --------------------------------------------------
    def connect_pair(self, dev: int = 0, max_polls: int = 1000):
        """listen -> (connect until non-NULL || accept until non-NULL), as a proxy thread would."""
        rc, handle, lcomm = self.listen(dev)
        assert rc == ncclSuccess
        send = recv = None
        for _ in range(max_polls):
            if send is None:
                rc, s = self.connect(dev, handle)
                assert rc == ncclSuccess
                send = s
            if recv is None:
                rc, r = self.accept(lcomm)
                assert rc == ncclSuccess
                recv = r
            if send is not None and recv is not None:
                return lcomm, send, recv
        raise RuntimeError("connection did not come up")

    def wait(self, request, max_polls: int = 10_000_000):
        """Poll test() until done; returns the reported size."""
        for _ in range(max_polls):
            rc, done, size = self.test(request)
            if rc != ncclSuccess:
                raise RuntimeError(f"test failed with ncclResult {rc}")
            if done:
                return size
        raise TimeoutError("request did not complete")

    # ---- control surface ------------------------------------------------------------------------------
    def reconfigure(self, **env) -> None:
        """Re-reads the NCCL_* parameters: sets the given environment variables (None unsets), then
        reset + init.  Only legal while no connection is open."""
        for k, v in env.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = str(v)
        rc = self.lib.fl_net_reset()
        if rc != 0:
            raise RuntimeError("fl_net_reset refused: connections are still open")
        assert self.init() == ncclSuccess

    def set_credits(self, credits) -> None:
        arr = (C.c_uint32 * len(credits))(*credits)
        assert self.lib.fl_net_set_credits(arr, len(credits)) == 0

    def comm_stats(self, comm):
        a, b, c = C.c_int64(), C.c_int64(), C.c_int64()
        assert self.lib.fl_net_comm_stats(comm, C.byref(a), C.byref(b), C.byref(c)) == 0
        return {"n_finished": a.value, "in_flight": b.value, "refreshes": c.value}

    def mask_stats(self, comm):
        m, n = C.c_uint32(), C.c_int64()
        assert self.lib.fl_net_mask_stats(comm, C.byref(m), C.byref(n)) == 0
        return {"mask": m.value, "refreshes": n.value}

    def free_requests(self, comm) -> int:
        return self.lib.fl_net_free_requests(comm)

    def launch_stats(self, comm):
        a, b = C.c_int64(), C.c_int64()
        assert self.lib.fl_net_launch_stats(comm, C.byref(a), C.byref(b)) == 0
        return {"launches": a.value, "batched_requests": b.value}

    def last_table(self, send_comm, max_rows: int = 4096):
        import numpy as np

        from .core import DESC_DTYPE, HDR_DTYPE
        rows = np.zeros(max_rows, dtype=DESC_DTYPE)
        hdr = np.zeros(1, dtype=HDR_DTYPE)
        n = self.lib.fl_net_last_table(send_comm, rows.ctypes.data_as(VP), max_rows, hdr.ctypes.data_as(VP))
        if n < 0:
            raise RuntimeError("fl_net_last_table failed")
        return rows[: min(n, max_rows)], hdr[0]

    def last_launch(self, comm, max_rows: int = 4096):
        """Segments, table and header of the last launch pair on the GPU that `comm` stages on."""
        import numpy as np

        from .core import DESC_DTYPE, HDR_DTYPE
        segs = (LaunchSeg * 8)()
        rows = np.zeros(max_rows, dtype=DESC_DTYPE)
        hdr = np.zeros(1, dtype=HDR_DTYPE)
        n = self.lib.fl_net_last_launch(comm, segs, 8, rows.ctypes.data_as(VP), max_rows, hdr.ctypes.data_as(VP))
        if n < 0:
            raise RuntimeError("fl_net_last_launch failed")
        out = [dict(channel=s.channel, first_row=s.first_row, n_rows=s.n_rows, n_req=s.n_req, epoch_bytes=s.epoch_bytes,
                    lane_base=list(s.lane_base)) for s in segs[:n]]
        total = sum(s["n_rows"] for s in out)
        return out, rows[:total], hdr[0]

    def flush(self, comm) -> None:
        assert self.lib.fl_net_flush(comm) == 0
