"""Child process of test_gpu_torch_hook.py: a DistributedDataParallel model on a one-rank RCCL process group with
cntk_amd.torch_hook.quantized_allreduce_hook registered, against the same model stepped without DDP whose gradients
go through a QuantizedGradientAggregator directly. Prints one JSON line."""
import json
import os
import sys

import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))


def main():
    import torch.distributed as dist
    from torch.nn.parallel import DistributedDataParallel

    from cntk_amd.torch_hook import QuantizedGradientAggregator, make_hook_state, quantized_allreduce_hook

    torch.cuda.set_device(0)
    try:
        dist.init_process_group("nccl", init_method="tcp://127.0.0.1:29517", rank=0, world_size=1)
    except Exception as e:  # no usable collective library or rendezvous on this machine
        print(json.dumps({"skipped": "process group could not be created: %r" % (e,)}), flush=True)
        return 0
    torch.manual_seed(1234)

    def make():
        return torch.nn.Sequential(torch.nn.Linear(300, 128), torch.nn.ReLU(), torch.nn.Linear(128, 64), torch.nn.ReLU(),
                                   torch.nn.Linear(64, 10)).cuda()

    plain = make()
    wrapped = make()
    wrapped.load_state_dict(plain.state_dict())
    ddp = DistributedDataParallel(wrapped, device_ids=[0])
    state = make_hook_state(None, nbits=1, zero_threshold_for_1bit=True, average=True)
    ddp.register_comm_hook(state, quantized_allreduce_hook)
    worst, steps = 0.0, 0
    for step in range(3):
        x = torch.randn(32, 300, device="cuda")
        y = torch.randint(0, 10, (32,), device="cuda")
        for m in (plain, ddp):
            m.zero_grad(set_to_none=True)
            torch.nn.functional.cross_entropy(m(x), y).backward()
        # fresh residuals on both sides every step: DistributedDataParallel regroups its buckets after the first
        # iteration, which starts the hook's residuals afresh, and the comparison is of one step's arithmetic
        state.reset_state()
        grads = [p.grad for p in plain.parameters()]
        QuantizedGradientAggregator(1, True).aggregate(grads)
        torch.cuda.synchronize()
        for p, q in zip(plain.parameters(), wrapped.parameters()):
            scale = float(p.grad.abs().max())
            worst = max(worst, float((p.grad - q.grad).abs().max()) / max(scale, 1e-30))
        steps += 1
        print("step", step, "worst relative difference", worst, flush=True)
    # the transport's two collectives as the aggregator calls them (one rank: every byte comes back to its sender)
    from cntk_amd.torch_hook import TorchDistributedTransport

    t = TorchDistributedTransport(None)
    send = torch.arange(4096, device="cuda", dtype=torch.int32).to(torch.uint8)
    recv, gathered = torch.zeros_like(send), torch.zeros_like(send)
    t.all_to_all(send, [send.numel()] * t.world_size, recv)
    t.all_gather(send, gathered)
    torch.cuda.synchronize()
    transport_ok = bool(torch.equal(recv, send) and torch.equal(gathered, send)) and t.world_size == 1 and t.rank == 0
    print(json.dumps({"steps": steps, "max_err": worst, "aggregators": len(state.aggregators), "transport_ok": transport_ok}), flush=True)
    dist.destroy_process_group()
    return 0


if __name__ == "__main__":
    sys.exit(main())
