"""Run as a script in a process of its own: one rank, one GPU, RCCL initialised with whatever
NCCL_NET_PLUGIN / LD_LIBRARY_PATH the caller set, one all-reduce.  RCCL loads the net plugin at
communicator creation and, to decide on GPU Direct, drives listen / connect / accept / regMr /
deregMr / close on every device the plugin reports; the caller reads RCCL's log."""
import os
import sys

import torch
import torch.distributed as dist


def main() -> int:
    os.environ.setdefault("MASTER_ADDR", "127.0.0.1")
    os.environ.setdefault("MASTER_PORT", "29533")
    dist.init_process_group("nccl", rank=0, world_size=1)
    x = torch.ones(1024, device="cuda")
    dist.all_reduce(x)
    torch.cuda.synchronize()
    print("allreduce", float(x.sum()), flush=True)
    dist.destroy_process_group()
    return 0


if __name__ == "__main__":
    sys.exit(main())
