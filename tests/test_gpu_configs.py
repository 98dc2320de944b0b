"""The five benchmark workloads of this path (speech DNN, ResNet-50, LSTM LM gradient sets, simulated 8-worker all-reduce), at their real shapes, through the C ABI. Needs an MI355X.

At full size the GPU chain runs freely on its own residual (gradients are generated on the device), every step is
checked through size-independent properties (conservation of the error feedback, codes consistent with the
stored header), and selected steps are checked against the CPU oracle on the very (gradient, residual-in) the GPU
saw at that step, downloaded from the device.
"""
import sys

import numpy as np
import pytest
import torch

import cntk_amd
import datagen
import oracle
import parity
from cntk_amd import Matrix, MatrixQuantizer, MatrixQuantizerImpl, QuantizedMatrix

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def np_of(m):
    return m.to_numpy()


def device_normal(gen, rows, cols, sigma):
    return Matrix(rows, cols, 0, torch.randn(rows * cols, generator=gen, device="cuda:0", dtype=torch.float32) * sigma)


def device_student_t3(gen, rows, cols, scale):
    n = rows * cols
    z = torch.randn(n, generator=gen, device="cuda:0", dtype=torch.float32)
    chi = torch.randn(3, n, generator=gen, device="cuda:0", dtype=torch.float32).square_().sum(0)
    return Matrix(rows, cols, 0, z / torch.sqrt(chi / 3.0) * scale)


def device_outliers(gen, rows, cols, sigma=0.01, frac=0.01, mult=50.0):
    n = rows * cols
    a = torch.randn(n, generator=gen, device="cuda:0", dtype=torch.float32) * sigma
    mask = torch.rand(n, generator=gen, device="cuda:0") < frac
    return Matrix(rows, cols, 0, torch.where(mask, a * mult, a))


def conservation_on_device(G, r_in_data, R, Out):
    """g + r_in == unquantize(q) + r_out up to the rounding of the two fp32 operations involved."""
    v = G.data + r_in_data
    back = Out.data
    diff = (v - (back + R.data)).abs()
    bound = 4e-7 * (v.abs() + back.abs()) + 1e-37
    bad = int((diff > bound).sum().item())
    assert bad == 0, "%d elements violate the conservation law" % bad


class Chain:
    """One gradient matrix with its carried residual, quantized and unquantized every step."""

    def __init__(self, rows, cols, nbits, zt):
        self.rows, self.cols, self.nbits, self.zt = rows, cols, nbits, zt
        self.mq = MatrixQuantizer(rows, cols, 0, False)
        self.Q = QuantizedMatrix(rows, cols, nbits, 0)
        self.Out = Matrix(rows, cols)

    def step(self, G, check_oracle, report):
        R = self.mq.GetResidualMatrix()
        r_in = R.data.clone()
        self.mq.QuantizeAsync(G, self.Q, self.zt)
        self.mq.UnquantizeAsync(self.Q, self.Out, add=False)
        self.mq.WaitUnquantizeAsyncDone()
        conservation_on_device(G, r_in, R, self.Out)
        if check_oracle:
            g = np_of(G)
            r0 = np.asfortranarray(r_in.cpu().numpy().reshape((self.rows, self.cols), order="F"))
            q = self.Q.to_numpy()
            parity.check_quantize(g, r0, q, np_of(R), self.nbits, self.zt, threads=16, report=report, strict=True)
            parity.check_unquantize(q, self.rows, self.cols, self.nbits, np_of(self.Out), threads=16)


# ---- config 1 ----------------------------------------------------------------------------------------


def test_config1_512x512_single_step():
    """512x512, N(0, 0.01^2) from seed, zero residual, one step, 1 bit, zeroThresholdFor1Bit off."""
    rows = cols = 512
    g = datagen.normal(datagen.case_seed(1), rows, cols, 0.01)
    qz = MatrixQuantizerImpl.Create(0, False)
    G, R, Q, Out = Matrix.from_numpy(g), Matrix(rows, cols), QuantizedMatrix(rows, cols, 1, 0), Matrix(rows, cols)
    qz.QuantizeAsync(G, R, Q, R, False)
    qz.WaitQuantizeAsyncDone()
    qz.UnquantizeAsync(Q, Out)
    qz.WaitUnquantizeAsyncDone()
    rep = parity.check_quantize(g, np.zeros_like(g, order="F"), Q.to_numpy(), np_of(R), 1, False, strict=True)
    parity.check_unquantize(Q.to_numpy(), rows, cols, 1, np_of(Out))
    assert Q.GetSize() == 36864
    say("config 1:", rep)
    rep.assert_fallback_at_most(0)


# ---- config 2 ----------------------------------------------------------------------------------------

# columns (of 27 checked steps x 23,656) allowed to rest on the float64 bounds instead of the oracle's
CONFIG2_FALLBACK_COLS = 0

SPEECH_DNN = [(429, 2048)] + [(2048, 2048)] * 6 + [(2048, 9304)] + [(2048, 1)] * 7 + [(9304, 1)]


@pytest.mark.parametrize("zt", [True, False], ids=["zeroThr", "meanThr"])
def test_config2_speech_dnn_100_steps(zt):
    """429-2048x7-9304 DNN gradient set, Student-t(3) x 1e-3, 1 bit, residual carried over 100 steps."""
    assert sum(r * c for r, c in SPEECH_DNN) == 45122648
    gen = torch.Generator(device="cuda:0")
    gen.manual_seed(datagen.case_seed(2))
    chains = [Chain(r, c, 1, zt) for r, c in SPEECH_DNN]
    rep = parity.Report()
    for step in range(100):
        if step % 10 == 0:
            say("config 2 zeroThr", zt, "step", step)
        for ch in chains:
            G = device_student_t3(gen, ch.rows, ch.cols, 1e-3)
            ch.step(G, step < 2 or step % 4 == 3, rep)  # the oracle sees steps 0, 1, 3, 7, 11 ... 99
    say("config 2:", rep)
    rep.assert_fallback_at_most(CONFIG2_FALLBACK_COLS)


# ---- config 3 ----------------------------------------------------------------------------------------


def resnet50_shapes():
    convs = [(147, 64)]
    def stage(cin, mid, cout, blocks):
        out = [(cin, mid), (9 * mid, mid), (mid, cout), (cin, cout)]  # first block + projection
        for _ in range(blocks - 1):
            out += [(cout, mid), (9 * mid, mid), (mid, cout)]
        return out
    convs += stage(64, 64, 256, 3) + stage(256, 128, 512, 4) + stage(512, 256, 1024, 6) + stage(1024, 512, 2048, 3)
    assert len(convs) == 53
    shapes = list(convs) + [(2048, 1000), (1000, 1)]
    for _, cout in convs:  # batch-norm scale and bias as column vectors
        shapes += [(cout, 1), (cout, 1)]
    return shapes


@pytest.mark.parametrize("nbits", [2, 4, 8])
def test_config3_resnet50_multibit(nbits):
    """ResNet-50 gradient set, N(0, 1e-4) with 1% outliers at 50x, mean-0 +/-4-sigma range quantizer."""
    shapes = resnet50_shapes()
    assert sum(r * c for r, c in shapes) == 25557032
    gen = torch.Generator(device="cuda:0")
    gen.manual_seed(datagen.case_seed(3, nbits))
    chains = [Chain(r, c, nbits, False) for r, c in shapes]
    rep = parity.Report()
    for step in range(3):
        say("config 3 nbits", nbits, "step", step)
        for ch in chains:
            ch.step(device_outliers(gen, ch.rows, ch.cols), True, rep)
    say("config 3:", rep)
    rep.assert_fallback_at_most(0)


# ---- config 4 ----------------------------------------------------------------------------------------


def test_config4_allreduce_full_shape():
    """8 simulated workers x 2048x9304, own residuals; 8 stripes of 2048x1163 reduced with stripe residuals."""
    rows, cols, k, nbits, zt = 2048, 9304, 8, 1, False
    gen = torch.Generator(device="cuda:0")
    gen.manual_seed(datagen.case_seed(4))
    workers = [MatrixQuantizer(rows, cols, 0, True) for _ in range(k)]
    Q = [QuantizedMatrix(rows, cols, nbits, 0) for _ in range(k)]
    S = [Matrix(rows, cntk_amd.stripe_range(cols, s, k)[1]) for s in range(k)]
    Qagg, Out = QuantizedMatrix(rows, cols, nbits, 0), Matrix(rows, cols)
    res_o = [np.zeros((rows, cols), np.float32, order="F") for _ in range(k)]
    sres_o = [np.zeros((rows, cntk_amd.stripe_range(cols, s, k)[1]), np.float32, order="F") for s in range(k)]
    qcol = oracle.qcol_bytes(nbits, rows)
    rep = parity.Report()
    for step in range(2):
        say("config 4 step", step)
        G = [device_normal(gen, rows, cols, 0.01) for _ in range(k)]
        # teacher forcing: the device starts every step from the oracle's residuals
        for w in range(k):
            workers[w].GetResidualMatrix().data.copy_(Matrix.from_numpy(res_o[w]).data)
        for s in range(k):
            S[s].data.copy_(Matrix.from_numpy(sres_o[s]).data)
        torch.cuda.synchronize()
        for w in range(k):
            workers[w].impl.SynchronizeWithMainStream()
            workers[w].QuantizeAsync(G[w], Q[w], zt)
        workers[k - 1].WaitQuantizeAsyncDone()
        torch.cuda.synchronize()
        q1 = [q.to_numpy() for q in Q]
        for s in range(k):
            start, n = cntk_amd.stripe_range(cols, s, k)
            stripes = [Q[w].ColumnSlice(start, n) for w in range(k)]
            workers[s].impl.StripeReduceAsync(stripes, s, S[s], stripes[s], zt)
        workers[k - 1].impl.WaitStripeReduceDone()
        torch.cuda.synchronize()
        for s in range(k):
            start, n = cntk_amd.stripe_range(cols, s, k)
            Qagg.ColumnSlice(start, n).buffer.copy_(Q[s].ColumnSlice(start, n).buffer)
        torch.cuda.synchronize()
        workers[0].impl.SynchronizeWithMainStream()
        workers[0].UnquantizeAsync(Qagg, Out)
        workers[0].WaitUnquantizeAsyncDone()
        torch.cuda.synchronize()

        gs = [np_of(g) for g in G]
        res_in = [r.copy(order="F") for r in res_o]
        sres_in = [s.copy(order="F") for s in sres_o]
        _, aggs_o, qagg_o, out_o = parity.oracle_allreduce_staged(gs, res_o, sres_o, nbits, zt, threads=16)
        qagg_g, out_g = Qagg.to_numpy(), np_of(Out)
        tainted = np.zeros(cols, dtype=bool)
        for w in range(k):
            parity.check_quantize(gs[w], res_in[w], q1[w], np_of(workers[w].GetResidualMatrix()), nbits, zt,
                                  threads=16, report=rep, strict=True)
            tainted |= rep.last_mismatch_cols
        for s in range(k):
            start, n = oracle.stripe_range(cols, s, k)
            q_copy = [q.copy() for q in q1]
            s_copy = sres_in[s].copy(order="F")
            agg = oracle.stripe_reduce(q_copy, s, rows, cols, nbits, s_copy, zt, threads=16)
            parity.check_quantize(agg, sres_in[s], qagg_g[start * qcol:(start + n) * qcol], np_of(S[s]), nbits, zt,
                                  threads=16, report=rep, strict=True)
            tainted[start:start + n] |= rep.last_mismatch_cols
        parity.check_unquantize(qagg_g, rows, cols, nbits, out_g, threads=16)
        worst, ntaint = parity.check_end_to_end(aggs_o, sres_in, qagg_g, [np_of(x) for x in S], out_g, qagg_o, out_o, rows,
                                                cols, nbits, zt, tainted, threads=16, report=rep)
        say("   aggregated gradient: max err %.3g of column scale; %d of %d columns hold a near-threshold flip"
            % (worst, ntaint, cols))
        assert ntaint <= cols // 100
    say("config 4:", rep)
    rep.assert_fallback_at_most(0)


# ---- config 5 ----------------------------------------------------------------------------------------

# of 11 checked steps x 116,896 columns
CONFIG5_FALLBACK_COLS = 8

LSTM_LM = [(100000, 512, 0.9), (1024, 4096, 0.0), (1024, 4096, 0.0), (1024, 4096, 0.0), (1024, 4096, 0.0),
           (512, 100000, 0.0)]


def test_config5_lstm_lm_zero_threshold_20_steps():
    """Embedding 100000x512 with 90% all-zero columns, 4 LSTM matrices 1024x4096, softmax 512x100000; 1 bit with
    zeroThresholdFor1Bit on, residual carried over 20 steps."""
    gen = torch.Generator(device="cuda:0")
    gen.manual_seed(datagen.case_seed(5))
    chains = [Chain(r, c, 1, True) for r, c, _ in LSTM_LM]
    rep = parity.Report()
    for step in range(20):
        say("config 5 step", step)
        for ch, (r, c, zero_frac) in zip(chains, LSTM_LM):
            G = device_normal(gen, r, c, 0.01)
            if zero_frac > 0:
                # a different 90% of the columns is silent at every step
                keep = (torch.rand(c, generator=gen, device="cuda:0") >= zero_frac).to(torch.float32)
                G.data.view(c, r).mul_(keep[:, None])
            ch.step(G, step < 2 or step % 2 == 1, rep)  # the oracle sees steps 0, 1, 3, 5 ... 19
    say("config 5:", rep)
    # only the 100000-row embedding columns that received a gradient (about 51 of 512 per step) are long enough for the
    # oracle's own fp32 sum to use up the tolerance
    rep.assert_fallback_at_most(CONFIG5_FALLBACK_COLS)
    # columns that never received a gradient keep lower = upper = 0 and all valid bits set
    z = Matrix(100000, 4)
    Qz = QuantizedMatrix(100000, 4, 1, 0)
    qz = MatrixQuantizerImpl.Create(0, False)
    qz.QuantizeAsync(z, Matrix(100000, 4), Qz, Matrix(100000, 4), True)
    qz.WaitQuantizeAsyncDone()
    w = oracle.words(Qz.to_numpy(), 100000, 4, 1)
    assert (w == 0xFFFFFFFF).all() and not np.any(oracle.headers(Qz.to_numpy(), 100000, 4, 1))
