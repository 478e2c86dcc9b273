"""Calls of the library on a stream that is under capture into a HIP graph are refused with an error before anything
is launched (every launching entry point asks hipStreamIsCapturing first).  Runs late in the collection order; the
capture here holds one library-free fill kernel of PyTorch, so the graph is not empty."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu


def test_library_calls_refuse_a_capturing_stream():
    from fly_amd import matmul
    from fly_amd.sblocal_attention import SBLocalPlan
    dev = torch.device('cuda:0')
    g = torch.Generator().manual_seed(0)
    B, H, L, E, mh, lc = 1, 1, 256, 64, 32, 64
    q, k, v = (torch.randn(B, L, H, E, generator=g).to(dev) for _ in range(3))
    P = torch.randn(mh, E, generator=g).to(dev)
    plan = SBLocalPlan(B, H, L, L, E, mh, mh, torch.float32, dev, lc)
    out = torch.empty(B, L, H, E, device=dev)
    ln = torch.empty(B, H, L, device=dev)
    plan.run(q, k, v, P, None, lc, 1 / math.sqrt(E), out, ln)                  # eager: scratch, first-use set-up
    layout = torch.ones(1, 2, 2, dtype=torch.long)
    sdd = matmul(layout, 32, 'sdd', trans_b=True)
    a = torch.randn(1, 1, 64, 64, generator=g).bfloat16().to(dev)
    sdd(a, a)
    torch.cuda.synchronize()
    want = out.clone()

    filler = torch.zeros(16, device=dev)
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    errors = []
    with torch.cuda.stream(side):
        graph.capture_begin()
        try:
            filler.add_(1.0)
            for call in (lambda: plan.run(q, k, v, P, None, lc, 1 / math.sqrt(E), out, ln), lambda: sdd(a, a)):
                try:
                    call()
                    errors.append(None)
                except RuntimeError as e:
                    errors.append(str(e))
        finally:
            graph.capture_end()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    assert all(e is not None and 'graph capture' in e for e in errors), errors
    # nothing was launched by the refused calls, and the library works as before afterwards
    plan.run(q, k, v, P, None, lc, 1 / math.sqrt(E), out, ln)
    torch.cuda.synchronize()
    assert torch.equal(out, want)
