"""A guard against one way the compiler has broken the copy kernels: the unrolled paths of a block copy load U
16-byte vectors and then store them (once, or twice in the copies with two destinations), all inside one basic block.
The optimizer once sank the trailing stores of such a path into a block shared with the predicated loop beside it, and
the generated code left the index of the first sunk store unwritten on the unrolled path: a lost store, or a wild one.
A marker at the end of each path of the two-destination copy (an empty asm statement that names the path) keeps the
tails apart.  The device code of fl_copy.hip is compiled to assembly (no GPU needed); every basic block that issues
four or more 16-byte loads must hold as many stores, and every block that carries the marker of an unrolled
two-destination path must hold its U loads and 2 U stores."""
import collections
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_every_unrolled_copy_block_holds_its_stores(tmp_path):
    from fuselink_amd import build
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("no hipcc")
    out = tmp_path / "fl_copy.s"
    flags = [f for f in build.FLAGS if f not in ("-shared", "-fPIC", "-pthread")]
    cmd = [hipcc, *flags, "-I" + os.path.join(ROOT, "include"), "-I" + build.CSRC, "-S", "--cuda-device-only", "-o", str(out),
           os.path.join(build.CSRC, "fl_copy.hip")]
    res = subprocess.run(cmd, capture_output=True, text=True, timeout=900)
    assert res.returncode == 0, res.stderr[-3000:]
    shapes = collections.Counter()
    odd = []
    fn, block, loads, stores, marked = None, None, 0, 0, 0

    def flush():
        nonlocal loads, stores, marked
        if loads >= 4 or marked:
            shapes[(loads, stores, marked)] += 1
            if (marked and (loads, stores) != (marked, 2 * marked)) or (not marked and stores != loads):
                odd.append((fn, block, loads, stores, marked))
        loads = stores = marked = 0

    for line in open(out):
        t = line.strip()
        m = re.match(r"^(_Z\S+|fl_\S+):", line)
        if m:
            flush()
            fn, block = m.group(1), "entry"
        elif re.match(r"^\.LBB\d+_\d+:", line):
            flush()
            block = t.split(":")[0]
        elif t.startswith(";"):
            m2 = re.match(r"^; two-destination copy, (\d+) vectors per thread", t)
            if m2:
                marked = int(m2.group(1))
            continue
        elif "load_dwordx4" in t:
            loads += 1
        elif "store_dwordx4" in t:
            stores += 1
        elif t.startswith(("s_cbranch", "s_branch", "s_endpgm", "s_setpc")):
            flush()
    flush()
    assert not odd, f"blocks whose stores were moved away from their loads: {odd[:10]}"
    # the shapes the source asks for: 4, 8 or 16 vectors to one destination, 8 or 16 to two (marked)
    assert set(shapes) <= {(4, 4, 0), (8, 8, 0), (16, 16, 0), (8, 16, 8), (16, 32, 16)}, shapes
    assert shapes[(8, 16, 8)] > 0 and shapes[(16, 32, 16)] > 0 and shapes[(8, 8, 0)] > 0
