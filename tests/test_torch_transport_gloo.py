"""The torch.distributed transport of the PyTorch aggregator on several ranks: gloo on the CPU, one child process per
rank. Checks that the all-to-all and the all-gather place every worker's slot where QuantizedGradientAggregator (and the
in-process group, whose exchange the GPU tests check against the oracle) expects it. No GPU needed."""
import json
import os
import socket
import subprocess
import sys

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))


def free_port():
    with socket.socket() as s:
        s.bind(("127.0.0.1", 0))
        return s.getsockname()[1]


@pytest.mark.parametrize("world,slot", [(2, 4096), (3, 1000)])
def test_transport_places_slots(world, slot):
    port = free_port()
    procs = [subprocess.Popen([sys.executable, "-u", os.path.join(HERE, "transport_gloo_worker.py"), str(r), str(world), str(port),
                               str(slot)], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True) for r in range(world)]
    outs = []
    try:
        for p in procs:
            outs.append(p.communicate(timeout=180))
    finally:
        for p in procs:
            if p.poll() is None:
                p.kill()
    for r, (p, (out, err)) in enumerate(zip(procs, outs)):
        lines = [ln for ln in out.splitlines() if ln.startswith("{")]
        assert p.returncode == 0 and lines, (r, out[-1000:], err[-2000:])
        assert json.loads(lines[-1]) == {"rank": r, "ok": True}
