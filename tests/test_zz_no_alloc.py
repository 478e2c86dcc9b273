"""The allocation-free variant of the fused Scatterbrain-local forward (flyhip_sblocal_fwd_static, whose
partial outputs live in an array inside the library) against flyhip_sblocal_fwd with a caller-allocated
workspace: same kernels, same order of operations, so the results must be bit-identical.  Two calls in a
row, the second on a smaller problem (it sees the first call's leftovers in the shared array)."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu


def _inputs(B, T, H, E, mh, seed, dtype):
    from oracle import sblocal as osb
    g = torch.Generator().manual_seed(seed)
    q, k, v = (torch.randn(B, T, H, E, generator=g) * (E ** -0.25 if i < 2 else 1.0) for i in range(3))
    P = osb.gaussian_orthogonal_random_matrix(mh, E, generator=g)
    return q.to(dtype), k.to(dtype), v.to(dtype), P


def _both(B, T, H, E, mh, lc, seed, dtype, lens=None):
    from fly_amd.sblocal_attention import SBLocalPlan
    from oracle import sblocal as osb
    dev = torch.device('cuda:0')
    q, k, v, P = _inputs(B, T, H, E, mh, seed, dtype)
    qd, kd, vd, Pd = (x.to(dev) for x in (q, k, v, P))
    ld = None if lens is None else torch.tensor(lens, device=dev)
    plan = SBLocalPlan(B, H, T, T, E, mh, mh, dtype, dev, lc)
    t = 1 / math.sqrt(E)
    outs = []
    for static in (False, True):
        out = torch.full((B, T, H, E), float('nan'), device=dev, dtype=dtype)
        ln = torch.full((B, H, T), float('nan'), device=dev)
        plan.run_keys(qd, kd, vd, Pd, ld, t)
        before = torch.cuda.memory_stats(dev)['allocation.all.allocated']
        if static:
            if plan.part_ws is not None:
                plan.part_ws.fill_(float('nan'))       # the static variant must not depend on it
            plan.run_queries_static(qd, kd, vd, Pd, ld, lc, t, out, ln)
        else:
            plan.run_queries(qd, kd, vd, Pd, ld, lc, t, out, ln)
        assert torch.cuda.memory_stats(dev)['allocation.all.allocated'] == before
        torch.cuda.synchronize()
        outs.append((out.cpu(), ln.cpu()))
    (o0, l0), (o1, l1) = outs
    assert torch.equal(o0, o1) and torch.equal(l0, l1)
    ref_out, ref_ln = osb.sblocal_attention(q.double(), k.double(), v.double(), P.double(), lc,
                                            key_lengths=None if lens is None else torch.tensor(lens))
    tol = 1e-4 if dtype == torch.float32 else 2e-2
    err = float((o1.double() - ref_out).abs().max() / ref_out.abs().max())
    assert err <= tol, err
    return plan.n_parts


def test_static_scratch_matches_workspace_variant():
    # BASELINE config 1 (five parts per query tile: 8.7 MB of partials), then a smaller ragged problem with
    # key lengths that also runs in parts, then bf16 and a one-part problem (no scratch at all)
    print('case config1', flush=True)
    assert _both(2, 3136, 1, 64, 64, 512, seed=0, dtype=torch.float32) > 1
    print('case small', flush=True)
    assert _both(2, 700, 2, 64, 32, 200, seed=1, dtype=torch.float32, lens=[700, 333]) > 1
    print('case bf16', flush=True)
    _both(1, 1024, 2, 64, 64, 256, seed=2, dtype=torch.bfloat16)
    print('case one part', flush=True)
    assert _both(64, 784, 1, 64, 64, 256, seed=3, dtype=torch.float32) == 1


def test_static_scratch_rejects_oversized_problems():
    from fly_amd.sblocal_attention import SBLocalPlan
    dev = torch.device('cuda:0')
    B, T, H, E, mh, lc = 4, 8192, 2, 64, 64, 512
    plan = SBLocalPlan(B, H, T, T, E, mh, mh, torch.float32, dev, lc, n_parts=4)      # 4*2*128*4*64*69 floats > 4 Mi
    q = torch.zeros(B, T, H, E, device=dev)
    P = torch.zeros(mh, E, device=dev)
    out, ln = torch.empty_like(q), torch.empty(B, H, T, device=dev)
    with pytest.raises(RuntimeError, match='built-in scratch'):
        plan.run_queries_static(q, q, q, P, None, lc, 0.125, out, ln)
