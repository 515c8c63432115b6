"""The device entry points under HIP graph capture: they allocate nothing, never synchronise and take their stream as an
argument, so a chain of them can be captured once and replayed.  Every replay is checked against the eager result of the
same inputs, with eager work and synchronisation between the replays."""
import numpy as np
import pytest
import torch

from neurotensor_amd import _lib
from neurotensor_amd import functional as F

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def setup_module(module):
    assert torch.cuda.is_available(), "GPU tests need a visible MI355X"
    _lib.load()


def _chain(x16, w16, b16, x32, w32, img, ker, xs, xodd, wodd):
    """A small model step touching every kernel family: DMA-fed 16-bit GEMM with bias, fp32 MFMA GEMM, the streaming
    (m <= 32) kernel, split-K, the padded-copy form, implicit-GEMM convolution and its gradients, the clamp epilogue and relu_
    in place."""
    y16 = F.linear(x16, w16, b16)                                   # [512, 1024] x [1024, 2048] + bias, bf16
    y32 = F.matmult(x32, w32, None, False, True)                    # fp32, transpose_b: 32-wide tiles, k split over the wavefronts
    yr = F.linear_relu(x16, w16, b16)                               # Linear -> ReLU in one launch
    y32r = F.relu_(F.matmult(x32, w32, None, False, True))          # relu_ on device memory
    ysk = F.matmult(xs, w16)                                        # 8 rows: streaming kernel
    ysp = F.matmult(y16[:256].contiguous(), w16, None, False, True)  # [256, 2048] x [2048, 1024]: split along k
    conv = F.conv2d(img, ker, padding=1)
    dimg, dker = F.conv2d_backward(img, ker, conv, padding=1)
    yodd = F.matmult(xodd, wodd)                                    # k = 1001: padded copy of A, B read in place + its last k-rows copied
    return y16, y32, ysk, ysp, conv, dimg, dker, yr, y32r, yodd


def test_capture_and_replay():
    torch.manual_seed(3)
    mk = lambda *s, dt=torch.float32, sc=1.0: (torch.randn(*s, device=DEV) * sc).to(dt)
    static = [mk(512, 1024, dt=torch.bfloat16, sc=0.1), mk(1024, 2048, dt=torch.bfloat16, sc=0.1), mk(2048, dt=torch.bfloat16),
              mk(300, 700), mk(260, 700), mk(4, 16, 20, 20), mk(8, 16, 3, 3, sc=0.1), mk(8, 1024, dt=torch.bfloat16, sc=0.1),
              mk(1304, 1001, dt=torch.bfloat16, sc=0.1), mk(1001, 1712, dt=torch.bfloat16, sc=0.1)]
    # warm up outside capture (first launches set kernel attributes)
    _chain(*static)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = _chain(*static)
    for rep in range(4):
        fresh = [torch.randn_like(t.float()).mul_(0.1 if t.dtype == torch.bfloat16 else 1.0).to(t.dtype) for t in static]
        for s, f in zip(static, fresh):
            s.copy_(f)
        graph.replay()
        torch.cuda.synchronize()
        got = [o.clone() for o in outs]
        # eager work between replays: the same chain on copies of the inputs
        want = _chain(*[f.clone() for f in fresh])
        torch.cuda.synchronize()
        for i, (g, w) in enumerate(zip(got, want)):
            assert torch.equal(g, w), (rep, i, (g.float() - w.float()).abs().max().item())
