"""fuselink_amd -- MI355X (gfx950) implementation of FuseLink's chunk split, chunk-to-lane
scheduling and staging-window striping / reassembly, behind the NCCL net-plugin ABI.

The compute lives in ``lib/libnccl-net-fuselink.so`` (hand-written HIP); this package is the thin
host mirror used by the tests, the smoke check and the benchmark.  Submodules import torch lazily
so that ``import fuselink_amd`` stays cheap."""

__all__ = ["build", "core", "plugin"]
