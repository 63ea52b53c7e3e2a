"""The entry points can be recorded into a HIP graph and replayed: one training step of a dense layer
(forward, backward, SGD update) plus an attention block and the operators next to them is captured once and
replayed on new inputs; every replay must equal the eager calls bit for bit.  This is what replaces the
reference's own record-and-replay of math calls (local_objects/vexectracer.cpp:586-1190, which re-issues the
recorded raw-pointer calls): the calls keep no state besides the library scratch, which the first eager run
has already sized, and clear memory with fill kernels rather than memset nodes.

PyTorch supplies the capture machinery (stream, graph object) and device memory here, nothing else.  The
body runs in a process of its own that imports torch BEFORE the library touches the GPU: torch brings its own
copy of the HIP runtime, and in a process where another copy is already initialised it finds no device."""
import os
import subprocess
import sys

import pytest


@pytest.mark.gpu
def test_training_step_graph_replays_equal_eager():
    out = subprocess.run([sys.executable, "-u", os.path.abspath(__file__)], capture_output=True, text=True, timeout=280)
    assert out.returncode == 0, out.stdout[-3000:] + out.stderr[-3000:]
    assert "graph replays equal eager" in out.stdout


def _body():
    import torch
    import numpy as np  # noqa: F401
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    from util import ko, rel_fro, REL_FRO_TOL
    from deep_learning_framework_amd import kai
    from deep_learning_framework_amd.kai import ACT, VMath

    kai.load()
    kai.set_device(0)
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev).manual_seed(5)
    ndat, xvec, yvec = 256, 1024, 1024                      # the product is cut along K: uses the library scratch
    nbat, T, nhead, D = 2, 64, 4, 16
    nvec = nhead * D
    t = lambda *shape: torch.empty(shape, device=dev)
    x, w0, b0, gy = t(ndat, xvec), t(yvec, xvec), t(yvec), t(ndat, yvec)
    w, b = t(yvec, xvec), t(yvec)
    y, pre, gx, gw, gb, work = t(ndat, yvec), t(ndat, yvec), t(ndat, xvec), t(yvec, xvec), t(yvec), t(ndat, yvec)
    q, k, v = t(nbat, T, nvec), t(nbat, T, nvec), t(nbat, T, nvec)
    p, o, ot = t(nbat, T, T, nhead), t(nbat, T, nvec), t(nbat, T, nvec)
    aff, st, rec = t(ndat, 4 * 256), t(ndat, 256), t(ndat, 256)
    lr = torch.tensor([0.05], device=dev)
    coef = torch.tensor([0.25], device=dev)
    table = torch.tensor([[0, T * nvec, T * nvec], [2, T * D, D], [1, D, nvec], [3, 1, 1]], dtype=torch.int32, device=dev)
    P = lambda a: a.data_ptr()

    def new_inputs(seed):
        gen.manual_seed(seed)
        x.normal_(generator=gen)
        gy.normal_(generator=gen).mul_(0.01)
        for a in (q, k, v):
            a.normal_(generator=gen)
        w.copy_(w0)
        b.copy_(b0)

    def step():
        VMath.dense_forward(0, P(y), P(pre), P(w), P(b), P(x), yvec, ndat, xvec, ACT["relu"], None)
        VMath.dense_backward(0, P(gx), P(gw), P(gb), P(work), P(gy), P(w), P(x), P(pre), yvec, ndat, xvec, ACT["relu"], None,
                             False)
        VMath.subtract_param_grad(0, P(w), P(gw), yvec * xvec, P(lr))
        VMath.subtract_param_grad(0, P(b), P(gb), yvec, P(lr))
        VMath.mult_on_heads(0, P(p), P(k), P(q), nbat, T, nvec, nhead, D, P(coef))
        VMath.set_mh_attention_mask(0, P(p), nbat, T, nhead, True)
        VMath.softmax_direct_on_axis(0, P(p), nbat * T, T, nhead)
        VMath.mix_values(0, P(o), P(p), P(v), nbat, T, nvec, nhead, D)
        VMath.transpose(0, P(ot), P(o), P(table), 4, o.numel())
        VMath.set_zero(0, P(aff), aff.numel() * 4)
        VMath.matmul(0, P(aff), P(w), P(y), yvec, ndat, xvec, True)
        VMath.lstm_process(0, P(rec), P(st), None, P(aff), ndat, 256, xvec)

    outputs = (y, gx, gw, gb, w, b, p, o, ot, rec, st)
    gen.manual_seed(1)
    w0.uniform_(-0.03, 0.03, generator=gen)
    b0.normal_(generator=gen)
    stream = torch.cuda.Stream()
    try:
        kai.set_stream(stream.cuda_stream)
        with torch.cuda.stream(stream):
            new_inputs(10)
            step()                                         # eager: sizes the library scratch before the capture
            stream.synchronize()
            # one check against the oracle, so that "equal to eager" means "right"
            ref = ko.activate(ko.add_bias(ko.matmul(w0.cpu().numpy(), x.cpu().numpy()), b0.cpu().numpy()), "relu")
            assert rel_fro(y.cpu().numpy(), ref) <= REL_FRO_TOL
            new_inputs(10)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                step()
            for seed in (11, 12, 13):
                new_inputs(seed)
                step()
                stream.synchronize()
                want = [a.clone() for a in outputs]
                for a in outputs:
                    a.fill_(float("nan"))
                new_inputs(seed)                           # same inputs, weights restored
                graph.replay()
                stream.synchronize()
                for a, ref_a in zip(outputs, want):
                    assert torch.equal(a, ref_a), "replay for seed %d differs from the eager calls" % seed
    finally:
        kai.set_stream(None)
    # A column sum over many rows of a narrow matrix cuts the rows into runs whose sums pass through the library
    # scratch; recorded on a stream that has no scratch yet (nothing may be allocated during a capture) it must take
    # its single launch instead of failing, and the replays must give the column sums.
    tall, sums = t(20000, 12), t(12)
    stream2 = torch.cuda.Stream()
    try:
        kai.set_stream(stream2.cuda_stream)
        with torch.cuda.stream(stream2):
            tall.normal_(generator=gen)
            stream2.synchronize()
            graph2 = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph2, stream=stream2):
                VMath.add_bias_backward_b(0, P(sums), P(tall), 20000, 12, False)
            for seed in (21, 22):
                gen.manual_seed(seed)
                tall.normal_(generator=gen)
                sums.fill_(float("nan"))
                graph2.replay()
                stream2.synchronize()
                ref = tall.double().sum(0)
                assert float((sums.double() - ref).norm() / ref.norm()) <= REL_FRO_TOL
            VMath.add_bias_backward_b(0, P(sums), P(tall), 20000, 12, False)   # eager: the runs, through the scratch
            stream2.synchronize()
            assert float((sums.double() - ref).norm() / ref.norm()) <= REL_FRO_TOL
    finally:
        kai.set_stream(None)
    print("graph replays equal eager")


if __name__ == "__main__":
    _body()
