"""One end of random traffic between two processes over the plugin's shared-memory wire (NCCL_FUSELINK_WIRE=shm).

Both processes run `drive` on the same plan: a list of connections, each with a direction, a seed and the sizes of its
requests.  A process listens for the connections it receives on, connects for the ones it sends on, registers one buffer
per connection, and then posts receives, posts sends and tests requests in a seeded random order, several in flight on
every connection, until all have completed; what arrived is compared with the connection's seeded pattern, byte by byte,
including the bytes behind the last request.  The handles travel as hex lines over the child's standard streams.

Run as a module (`python -m tests.two_process_peer <plan.json>`) this is the child's end, role "b"."""
import ctypes as C
import json
import sys
import time

import numpy as np


def make_plan(seed, n_ab, n_ba, requests, max_bytes, chunk, inflight):
    """n_ab connections from role a to role b, n_ba the other way; sizes from empty to max_bytes, a third of them whole
    chunks, one oversized request per connection."""
    rng = np.random.default_rng(seed)
    conns = []
    for i in range(n_ab + n_ba):
        sizes = []
        for q in range(requests):
            kind = int(rng.integers(0, 6))
            if kind == 0:
                n = int(rng.integers(1, 9)) * chunk
            elif kind == 1:
                n = int(rng.integers(0, 64))
            else:
                n = int(rng.integers(0, max_bytes + 1))
            sizes.append(n)
        sizes[int(rng.integers(0, requests))] = int(max_bytes * 5 + int(rng.integers(0, chunk)))   # more than the windows hold
        conns.append({"sender": "a" if i < n_ab else "b", "seed": int(rng.integers(1, 1 << 30)), "sizes": sizes})
    return {"conns": conns, "inflight": inflight, "seed": int(seed)}


def drive(p, P, plan, role, read_line, write_line, deadline_s=90, peer_alive=None):
    """p: a NetPlugin already initialised with the wire's parameters.  Returns the number of requests completed."""
    import torch
    deadline = time.time() + deadline_s
    conns = plan["conns"]
    mine_recv = [i for i, c in enumerate(conns) if c["sender"] != role]
    mine_send = [i for i, c in enumerate(conns) if c["sender"] == role]
    # listen for what this side receives; the child's handles go first, then the parent's
    listens = {}
    for i in mine_recv:
        rc, handle, lcomm = p.listen(i % 2)
        assert rc == P.ncclSuccess
        listens[i] = (handle, lcomm)

    def send_handles():
        for i in mine_recv:
            write_line(listens[i][0].raw.hex())

    def read_handles():
        out = {}
        for i in mine_send:
            line = read_line().strip()
            assert len(line) == 2 * P.NCCL_NET_HANDLE_MAXSIZE, line[:200]
            out[i] = C.create_string_buffer(bytes.fromhex(line), P.NCCL_NET_HANDLE_MAXSIZE)
        return out

    if role == "b":
        send_handles()
        theirs = read_handles()
    else:
        theirs = read_handles()
        send_handles()
    scomm, rcomm = {}, {}
    while len(scomm) < len(mine_send) or len(rcomm) < len(mine_recv):     # both calls are non-blocking: take turns
        for i in mine_send:
            if i not in scomm:
                rc, c = p.connect(i % 2, theirs[i])
                assert rc == P.ncclSuccess
                if c:
                    scomm[i] = c
        for i in mine_recv:
            if i not in rcomm:
                rc, c = p.accept(listens[i][1])
                assert rc == P.ncclSuccess
                if c:
                    rcomm[i] = c
        assert time.time() < deadline, "connections were not established"
    bufs, mhs, offs = {}, {}, {}
    for i, c in enumerate(conns):
        total = sum(c["sizes"])
        offs[i] = np.concatenate([[0], np.cumsum(c["sizes"])]).astype(np.int64)
        if i in scomm:
            pattern = np.random.default_rng(c["seed"]).integers(1, 256, size=total, dtype=np.uint8)
            bufs[i] = torch.from_numpy(pattern).cuda() if total else torch.zeros(64, dtype=torch.uint8, device="cuda")
            rc, mhs[i] = p.regMr(scomm[i], bufs[i].data_ptr(), bufs[i].numel(), P.NCCL_PTR_CUDA)
        else:
            bufs[i] = torch.zeros(total + 64, dtype=torch.uint8, device="cuda")
            rc, mhs[i] = p.regMr(rcomm[i], bufs[i].data_ptr(), bufs[i].numel(), P.NCCL_PTR_CUDA)
        assert rc == P.ncclSuccess
    torch.cuda.synchronize()
    rng = np.random.default_rng(plan["seed"] + (1 if role == "b" else 0))
    nxt = {i: 0 for i in range(len(conns)) if i in scomm or i in rcomm}
    out = {i: [] for i in nxt}            # requests in flight, oldest first: (request, index)
    completed = 0
    want = sum(len(conns[i]["sizes"]) for i in nxt)
    K = plan["inflight"]
    turns = 0
    while completed < want:
        turns += 1
        if turns % 4096 == 0:
            assert time.time() < deadline, f"role {role}: {completed} of {want} requests after {deadline_s} s"
            assert peer_alive is None or peer_alive(), "the other process has gone"
        i = int(rng.choice(list(nxt)))
        sizes = conns[i]["sizes"]
        act = int(rng.integers(0, 3))
        if act < 2 and nxt[i] < len(sizes) and len(out[i]) < K:
            q = nxt[i]
            if i in scomm:
                rc, req = p.isend(scomm[i], bufs[i].data_ptr() + int(offs[i][q]), sizes[q], q, mhs[i])
            else:
                rc, req = p.irecv(rcomm[i], [bufs[i].data_ptr() + int(offs[i][q])], [sizes[q]], [q], [mhs[i]])
            assert rc == P.ncclSuccess, (role, i, q, rc)
            if req:                       # none yet: the receive has not been posted, or the refresh gate holds it back
                out[i].append((req, q))
                nxt[i] += 1
        elif out[i]:
            req, q = out[i][0]            # in posting order, as NCCL's proxy tests them
            rc, done, got = p.test(req)
            assert rc == P.ncclSuccess, (role, i, q, rc)
            if done:
                if i in rcomm:
                    assert got == sizes[q], (role, i, q, got, sizes[q])
                out[i].pop(0)
                completed += 1
    torch.cuda.synchronize()
    for i in mine_recv:
        c = conns[i]
        total = sum(c["sizes"])
        exp = np.random.default_rng(c["seed"]).integers(1, 256, size=total, dtype=np.uint8)
        back = bufs[i].cpu().numpy()
        assert np.array_equal(back[:total], exp), f"connection {i}: received bytes differ from what was sent"
        assert not back[total:].any(), f"connection {i}: bytes behind the last request were touched"
    # both sides have everything: say so, wait for the other, then take the connections down
    write_line("received")
    assert read_line().strip() == "received"
    for i in scomm:
        assert p.deregMr(scomm[i], mhs[i]) == P.ncclSuccess and p.closeSend(scomm[i]) == P.ncclSuccess
    write_line("closed")
    assert read_line().strip() == "closed"
    for i in rcomm:
        assert p.deregMr(rcomm[i], mhs[i]) == P.ncclSuccess
        assert p.closeRecv(rcomm[i]) == P.ncclSuccess and p.closeListen(listens[i][1]) == P.ncclSuccess
    return completed


def main():
    from fuselink_amd import plugin as P
    plan = json.loads(sys.argv[1])
    p = P.NetPlugin(8)
    assert p.init() == P.ncclSuccess

    def write_line(s):
        sys.stdout.write(s + "\n")
        sys.stdout.flush()

    n = drive(p, P, plan, "b", sys.stdin.readline, write_line)
    write_line(f"peer ok {n}")


if __name__ == "__main__":
    main()
