"""The quantized gradient all-reduce as a gradient-compression step for PyTorch-ROCm.

Dataflow of AllReduceDistGradAggregator::AggregateGradientsImpl (Source/1BitSGD/AllReduceDistGradAggregator.h:268-531)
and of the v2 QuantizedDistributedCommunicator (QuantizedAggregate, Source/1BitSGD/QuantizedDistributedCommunicator.h:286-520)
on a set of torch gradient tensors, with every packed buffer resident on the device:

  1. every gradient is quantized with its error-feedback residual, stripe by stripe, straight into the send buffer
     (one batched launch for the whole set, one per element type),
  2. the packed stripes change hands (all-to-all: worker r's stripe s goes to worker s),
  3. the owner of a stripe decodes and sums the K packed stripes and requantizes the sum with its stripe residual
     (one batched launch),
  4. the requantized stripes change hands (all-gather),
  5. every worker unquantizes all stripes into its gradients (one batched launch).

The exchange is behind a small transport interface: `LocalTransport` (one worker), `InProcessTransport` (K workers in
one process on one GPU, for tests and timing) and `TorchDistributedTransport` (torch.distributed; RCCL on ROCm).
All kernels are issued on torch's current stream, so no host synchronisation is needed around them.

A tensor of shape (d0, d1, ...) is the column-major matrix with d0 columns of d1*... rows (a Linear weight [out, in]:
one column per output unit; a convolution [Cout, Cin, kH, kW]: [Cin*kH*kW x Cout]); vectors are single columns, as the
reference's bias parameters are.
"""
import torch

from . import (Matrix, MatrixQuantizerImpl, QuantizedMatrix, QuantizerLogicError, _fn, qcol_bytes, stripe_range)


def matrix_view(t):
    """Zero-copy column-major Matrix over a contiguous float32 / float64 device tensor."""
    if not t.is_cuda or t.dtype not in (torch.float32, torch.float64):
        raise QuantizerLogicError("gradient tensors must be float32 or float64 device tensors (got %s on %s)" % (t.dtype, t.device))
    if not t.is_contiguous():
        raise QuantizerLogicError("gradient tensors must be contiguous")
    cols = t.shape[0] if t.dim() >= 2 else 1
    return Matrix(t.numel() // max(cols, 1), cols, t.device.index, t.detach().view(-1))


def stripe_layout(shapes, world_size, nbits):
    """Where every packed stripe sits in a per-worker slot of the exchange buffers.

    shapes: (rows, cols, torch dtype) per gradient matrix. Returns (stripes, rel, slot): stripes[s][i] = (first column,
    columns) of matrix i that worker s owns (GetStripeForNode, Source/1BitSGD/AllReduceDistGradAggregator.h:56-65);
    rel[s][i] = byte offset of that packed stripe inside worker s's slot, 8-byte aligned (a packed column of doubles
    starts with two doubles); slot = bytes per slot, the largest worker's need, the same for all so that one size serves
    the all-to-all and the all-gather."""
    stripes = [[stripe_range(cols, s, world_size) for (_, cols, _) in shapes] for s in range(world_size)]
    rel, need = [], []
    for s in range(world_size):
        off, row = 0, []
        for i, (rows, _, dt) in enumerate(shapes):
            row.append(off)
            off += (stripes[s][i][1] * qcol_bytes(nbits, rows, dt) + 7) // 8 * 8
        rel.append(row)
        need.append(off)
    return stripes, rel, max(max(need), 8)


def stripe_residue_numel(t, rank, world_size):
    """Elements of the stripe residual that worker `rank` keeps for gradient tensor t (rows times its stripe's columns)."""
    cols = t.shape[0] if t.dim() >= 2 else 1
    return (t.numel() // max(cols, 1)) * stripe_range(cols, rank, world_size)[1]


class LocalTransport:
    """One worker: nothing changes hands (the aggregator never calls a transport of one worker)."""
    rank, world_size = 0, 1


class TorchDistributedTransport:
    """torch.distributed over the given process group (backend "nccl" is RCCL on ROCm)."""

    def __init__(self, process_group=None):
        import torch.distributed as dist
        self._dist, self._pg = dist, process_group
        self.rank, self.world_size = dist.get_rank(process_group), dist.get_world_size(process_group)

    def all_to_all(self, send, send_splits, recv):
        mine = send_splits[self.rank]
        self._dist.all_to_all_single(recv, send, [mine] * self.world_size, list(send_splits), group=self._pg)

    def all_gather(self, mine, gathered):
        self._dist.all_gather_into_tensor(gathered, mine, group=self._pg)


class InProcessTransport:
    """K workers in one process on one device. The workers' calls are collected and carried out by
    InProcessGroup, which steps all workers through the phases together."""

    def __init__(self, group, rank):
        self._group, self.rank, self.world_size = group, rank, group.world_size

    def all_to_all(self, send, send_splits, recv):
        self._group._posted[self.rank] = (send, send_splits, recv)

    def all_gather(self, mine, gathered):
        self._group._posted[self.rank] = (mine, gathered)


class QuantizedGradientAggregator:
    """One worker's side of the quantized all-reduce for a fixed list of gradient tensors.

    Residuals (one per gradient, one per owned stripe) live as long as the object and are created, zeroed, at the
    first call (ResetState, Source/1BitSGD/AllReduceDistGradAggregator.h:67-147). Gradients are summed over the
    workers as in the reference; pass average=True to divide by the number of workers afterwards (torch's
    DistributedDataParallel convention).
    """

    def __init__(self, nbits=1, zero_threshold_for_1bit=True, transport=None, average=False, residues=None, stripe_residues=None):
        """residues / stripe_residues: caller-owned residual tensors, as the v2 communicator takes them from its learner
        (QuantizedAggregateInPlace, Source/1BitSGD/QuantizedDistributedCommunicator.h:51-62): one per gradient, of the
        gradient's size, and one per gradient of the size of this worker's stripe (stripe_residue_numel). They are updated in
        place; without them the aggregator creates its own, zeroed."""
        self.nbits, self.zt, self.average = int(nbits), bool(zero_threshold_for_1bit), bool(average)
        self.transport = transport if transport is not None else LocalTransport()
        self._given = (residues, stripe_residues)
        self._geom = None
        self._plan = None

    def _adopt(self, given, grads, numels, what):
        """The caller's residual tensors as flat views, checked against what the gradients need."""
        if len(given) != len(grads):
            raise QuantizerLogicError("%s: one tensor per gradient" % what)
        out = []
        for t, g, n in zip(given, grads, numels):
            if t.device != g.device or t.dtype != g.dtype or t.numel() != n or not t.is_contiguous():
                raise QuantizerLogicError("%s: a contiguous tensor of %d elements of %s on %s is needed" % (what, n, g.dtype, g.device))
            out.append(t.detach().view(-1))
        return out

    # ---- set-up -------------------------------------------------------------------------------------

    def _setup(self, grads):
        t = self.transport
        W, me = t.world_size, t.rank
        dev = grads[0].device
        if any(g.device != dev for g in grads):
            raise QuantizerLogicError("all gradients of one aggregator must live on one device")
        self._impl = MatrixQuantizerImpl(dev.index, False)
        shapes = []
        for g in grads:
            m = matrix_view(g)
            shapes.append((m.rows, m.cols, g.dtype, qcol_bytes(self.nbits, m.rows, g.dtype)))
        self._stripe, self._rel, self._slot = stripe_layout([(r, c, dt) for (r, c, dt, _) in shapes], W, self.nbits)
        u8 = dict(dtype=torch.uint8, device=dev)
        self._send = torch.zeros(W * self._slot, **u8)
        self._recv = torch.zeros(W * self._slot, **u8) if W > 1 else None
        self._mine = torch.zeros(self._slot, **u8)
        self._gathered = torch.zeros(W * self._slot, **u8) if W > 1 else None
        stripe_numels = [shapes[i][0] * self._stripe[me][i][1] for i in range(len(grads))]
        if self._given[0] is not None:
            self._residual = self._adopt(self._given[0], grads, [g.numel() for g in grads], "residues")
        else:
            self._residual = [torch.zeros(g.numel(), dtype=g.dtype, device=dev) for g in grads]
        if self._given[1] is not None:
            self._stripe_residual = self._adopt(self._given[1], grads, stripe_numels, "stripe_residues")
        else:
            self._stripe_residual = [torch.zeros(n, dtype=g.dtype, device=dev) for n, g in zip(stripe_numels, grads)]
        self._shapes = shapes
        self._geom = [(tuple(g.shape), g.dtype) for g in grads]
        self._any64 = any(g.dtype == torch.float64 for g in grads)

    def _packed(self, buf, slot, s, i):
        """The packed stripe of gradient i that worker s owns, inside slot `slot` of buf."""
        rows, _, dt, qcol = self._shapes[i]
        n = self._stripe[s][i][1]
        o = slot * self._slot + self._rel[s][i]
        return QuantizedMatrix(rows, n, self.nbits, buf.device.index, buf[o:o + n * qcol], dtype=dt)

    def reset_state(self):
        """Zeroes all residuals (what the reference does when a checkpoint is restored:
        Source/1BitSGD/QuantizedDataParallelDistributedLearner.h:78-91)."""
        if self._geom is not None:
            for r in self._residual + self._stripe_residual:
                r.zero_()

    # ---- the five phases ------------------------------------------------------------------------------

    def _items(self, grads, want64):
        """(quantize items, unquantize items) of the float32 (want64=False) or float64 gradients, stripe by stripe."""
        W = self.transport.world_size
        everything = self._mine if W == 1 else self._gathered
        q_items, u_items = [], []
        for s in range(W):
            for i, t in enumerate(grads):
                start, n = self._stripe[s][i]
                if n == 0 or (t.dtype == torch.float64) != want64:
                    continue
                g = matrix_view(t)
                res = Matrix(g.rows, g.cols, g.device_id, self._residual[i]).ColumnSlice(start, n)
                q_items.append((g.ColumnSlice(start, n), res, self._packed(self._send, s, s, i), res))
                u_items.append((self._packed(everything, s, s, i), g.ColumnSlice(start, n)))
        return q_items, u_items

    def _plan_for(self, grads):
        """The argument blocks of the batched calls, built once per placement of the gradients in memory (the buffers
        and residuals never move; DistributedDataParallel's bucket views and .grad tensors that are zeroed in place
        do not either). The blocks hold addresses only, so no gradient is kept alive between calls."""
        where = tuple(g.data_ptr() for g in grads)
        if self._plan is not None and self._plan["where"] == where:
            return self._plan
        P = MatrixQuantizerImpl
        q32, u32 = self._items(grads, False)
        q64, u64 = self._items(grads, True) if self._any64 else ([], [])
        self._plan = dict(where=where, q=[P.PrepareQuantizeBatch(q32), P.PrepareQuantizeBatch(q64)],
                          u=[P.PrepareUnquantizeBatch(u32), P.PrepareUnquantizeBatch(u64)])
        return self._plan

    def _plan_stripes(self):
        """The owner's stripe reductions: they touch the aggregator's own buffers only, so they are laid out once."""
        W, me = self.transport.world_size, self.transport.rank
        arrived = self._send if W == 1 else self._recv
        fused, fused64, tall = [], [], []
        for i, (rows, _, dt, _) in enumerate(self._shapes):
            n = self._stripe[me][i][1]
            if n == 0:
                continue
            # worker r's stripe arrived in slot r; the own stripe never left the send buffer
            stripes = [self._packed(self._send, me, me, i) if r == me else self._packed(arrived, r, me, i) for r in range(W)]
            sres = Matrix(rows, n, self._send.device.index, self._stripe_residual[i])
            item = (stripes, sres, self._packed(self._mine, 0, me, i), None)
            if not self._impl.StripeReduceTakes(rows, n, self.nbits, self.zt, dt):
                tall.append(item)
            elif dt == torch.float32:
                fused.append(item)
            else:
                fused64.append(item)
        P = MatrixQuantizerImpl
        self._s_fused, self._s_tall = [P.PrepareStripeReduceBatch(fused), P.PrepareStripeReduceBatch(fused64)], tall

    def quantize(self, grads):
        """Phase 1 (AllReduceDistGradAggregator.h:288-300)."""
        if self._geom is None:
            self._setup(grads)
            self._plan_stripes()
        if [(tuple(g.shape), g.dtype) for g in grads] != self._geom:
            raise QuantizerLogicError("the gradient list differs from the one this aggregator was set up for")
        self._impl.SetMainStream(torch.cuda.current_stream(grads[0].device).cuda_stream)
        self._current = (self._plan_for(grads), grads)
        for prepared in self._current[0]["q"]:
            self._impl.QuantizeBatchAsync(prepared, self.zt)

    def exchange_stripes(self):
        """Phase 2 (AllReduceDistGradAggregator.h:302-384: the stripes' sends and receives): fills the receive buffer."""
        W = self.transport.world_size
        if W > 1:
            self.transport.all_to_all(self._send, [self._slot] * W, self._recv)

    def reduce(self):
        """Phase 3 (AllReduceDistGradAggregator.h:365-436, 494)."""
        W, me = self.transport.world_size, self.transport.rank
        for prepared in self._s_fused:
            self._impl.StripeReduceBatchAsync(prepared, me, self.zt)
        for stripes, sres, out, _ in self._s_tall:
            # shapes the fused kernels do not take: the reference's own sequence of calls
            agg = Matrix(sres.rows, sres.cols, sres.device_id, dtype=sres.dtype)
            self._impl.UnquantizeAsync(stripes[me], agg, add=False)
            for r in range(W):
                if r != me:
                    self._impl.UnquantizeAsync(stripes[r], agg, add=True)
            self._impl.QuantizeAsync(agg, sres, out, sres, self.zt)

    def exchange_reduced(self):
        """Phase 4 (AllReduceDistGradAggregator.h:438-515: the aggregated stripes' sends and receives): fills the
        gather buffer."""
        if self.transport.world_size > 1:
            self.transport.all_gather(self._mine, self._gathered)

    def unquantize(self):
        """Phase 5 (AllReduceDistGradAggregator.h:517-522)."""
        W = self.transport.world_size
        plan, grads = self._current
        for prepared in plan["u"]:
            self._impl.UnquantizeBatchAsync(prepared, add=False)
        if self.average and W > 1:
            for g in grads:
                g.div_(W)
        self._current = None

    def aggregate(self, grads):
        """All five phases, in place on `grads`. Returns when everything is enqueued on torch's current stream."""
        self.quantize(grads)
        self.exchange_stripes()
        self.reduce()
        self.exchange_reduced()
        self.unquantize()


class InProcessGroup:
    """K aggregators in one process on one device, stepped through the phases together; stripes change hands as
    device-to-device copies on the current stream."""

    def __init__(self, world_size, nbits=1, zero_threshold_for_1bit=True, average=False):
        self.world_size = int(world_size)
        self._posted = [None] * self.world_size
        self.workers = [QuantizedGradientAggregator(nbits, zero_threshold_for_1bit, InProcessTransport(self, r), average)
                        for r in range(self.world_size)]

    def aggregate(self, grads_per_worker):
        K = self.world_size
        if len(grads_per_worker) != K:
            raise QuantizerLogicError("one gradient list per worker")
        for w, g in zip(self.workers, grads_per_worker):
            w.quantize(g)
        self.aggregate_after_quantize()

    def aggregate_after_quantize(self):
        """Phases 2 to 5 for all workers, once every worker's quantize() has been called."""
        K = self.world_size
        for w in self.workers:
            w.exchange_stripes()
        for r in range(K if K > 1 else 0):  # worker r's slot s goes to worker s's slot r
            send, splits, _ = self._posted[r]
            for s in range(K):
                if s != r:
                    recv = self._posted[s][2]
                    recv[r * splits[r]:(r + 1) * splits[r]].copy_(send[s * splits[s]:(s + 1) * splits[s]])
        for w in self.workers:
            w.reduce()
        for w in self.workers:
            w.exchange_reduced()
        for r in range(K if K > 1 else 0):
            mine, _ = self._posted[r]
            for s in range(K):
                gathered = self._posted[s][1]
                gathered[r * mine.numel():(r + 1) * mine.numel()].copy_(mine)
        for w in self.workers:
            w.unquantize()


class _HookState:
    """What `quantized_allreduce_hook` keeps between calls: one aggregator per gradient bucket."""

    def __init__(self, process_group=None, nbits=1, zero_threshold_for_1bit=True, average=True):
        self.process_group, self.nbits, self.zt, self.average = process_group, nbits, zero_threshold_for_1bit, average
        self.aggregators = {}

    def reset_state(self):
        for a in self.aggregators.values():
            a.reset_state()


def make_hook_state(process_group=None, nbits=1, zero_threshold_for_1bit=True, average=True):
    """State for `quantized_allreduce_hook`; average=True gives DistributedDataParallel's mean of the gradients."""
    return _HookState(process_group, nbits, zero_threshold_for_1bit, average)


def quantized_allreduce_hook(state, bucket):
    """Communication hook for torch.nn.parallel.DistributedDataParallel.register_comm_hook: every parameter's
    gradient in the bucket goes through the quantized all-reduce, each as its own matrix with its own residual.
    Buckets must keep their composition from step to step (DistributedDataParallel's do after its first iteration
    has rebuilt them; the aggregator of a bucket whose composition changed is set up again, residuals zeroed)."""
    grads = bucket.gradients()
    key = bucket.index()
    geom = [(tuple(g.shape), g.dtype) for g in grads]
    agg = state.aggregators.get(key)
    if agg is None or agg._geom != geom:
        import torch.distributed as dist
        transport = TorchDistributedTransport(state.process_group) if dist.is_initialized() and \
            dist.get_world_size(state.process_group) > 1 else LocalTransport()
        agg = state.aggregators[key] = QuantizedGradientAggregator(state.nbits, state.zt, transport, state.average)
    agg.aggregate(grads)
    fut = torch.futures.Future()
    fut.set_result(bucket.buffer())
    return fut
