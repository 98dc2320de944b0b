"""Child process of test_torch_transport_gloo.py: one rank of a gloo process group on the CPU. Runs the two collectives of
cntk_amd.torch_hook.TorchDistributedTransport exactly as QuantizedGradientAggregator calls them (equal slots, the send
buffer's slot s addressed to worker s) on byte patterns that name their sender and slot, and checks where every byte
arrived. Prints one JSON line."""
import json
import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))


def pattern(rank, slot_index, slot):
    """Bytes that identify (sender, slot, position)."""
    i = torch.arange(slot, dtype=torch.int64)
    return ((i * 7 + 31 * rank + 101 * slot_index + 3) % 251).to(torch.uint8)


def main():
    import torch.distributed as dist

    from cntk_amd.torch_hook import TorchDistributedTransport

    rank, world, port, slot = (int(a) for a in sys.argv[1:5])
    dist.init_process_group("gloo", init_method="tcp://127.0.0.1:%d" % port, rank=rank, world_size=world)
    t = TorchDistributedTransport(None)
    ok = t.rank == rank and t.world_size == world
    # phase 2: slot s of the send buffer goes to worker s, which finds worker r's stripe in slot r
    send = torch.cat([pattern(rank, s, slot) for s in range(world)])
    recv = torch.zeros(world * slot, dtype=torch.uint8)
    t.all_to_all(send, [slot] * world, recv)
    for r in range(world):
        ok = ok and bool(torch.equal(recv[r * slot:(r + 1) * slot], pattern(r, rank, slot)))
    # phase 4: every worker's reduced stripes, in rank order
    mine = pattern(rank, 99, slot)
    gathered = torch.zeros(world * slot, dtype=torch.uint8)
    t.all_gather(mine, gathered)
    for r in range(world):
        ok = ok and bool(torch.equal(gathered[r * slot:(r + 1) * slot], pattern(r, 99, slot)))
    print(json.dumps({"rank": rank, "ok": bool(ok)}), flush=True)
    dist.destroy_process_group()
    return 0


if __name__ == "__main__":
    sys.exit(main())
