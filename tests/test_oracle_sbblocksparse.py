"""Pins of the block-sparse Scatterbrain oracle (CPU): the restated op sequence against an
independent closed form, against explicit loops on a tiny case, and the invariants the algebra
fixes."""
import math

import torch

from conftest import rel_err
from oracle import sbblocksparse as osbb
from oracle import sblocal as osb


def _inputs(B, T, S, H, E, D, mh, seed):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, T, H, E, generator=g, dtype=torch.float64) * E ** -0.25
    k = torch.randn(B, S, H, E, generator=g, dtype=torch.float64) * E ** -0.25
    v = torch.randn(B, S, H, D, generator=g, dtype=torch.float64)
    P = osb.gaussian_orthogonal_random_matrix(mh, E, generator=g).double()
    return q, k, v, P


def _layout(H, p, r, seed, density=0.5):
    g = torch.Generator().manual_seed(seed)
    lay = (torch.rand(H, p, r, generator=g) < density).long()
    lay[:, torch.arange(p), torch.arange(p) % r] = 1            # no empty block-row
    return lay


def test_op_sequence_equals_closed_form():
    for (B, T, S, H, E, D, mh, block, seed) in [(2, 64, 64, 2, 16, 16, 8, 16, 0), (1, 96, 64, 3, 32, 24, 16, 32, 1)]:
        q, k, v, P = _inputs(B, T, S, H, E, D, mh, seed)
        layout = _layout(H, T // block, S // block, seed)
        out, ln = osbb.sbblocksparse_attention(q, k, v, P, layout, block)
        ref_out, ref_ln = osbb.dense_closed_form(q, k, v, P, layout, block)
        assert rel_err(out, ref_out) < 1e-10 and rel_err(ln, ref_ln) < 1e-10


def test_tiny_case_by_loops():
    B, T, S, H, E, D, mh, block = 1, 32, 32, 1, 4, 3, 2, 16
    q, k, v, P = _inputs(B, T, S, H, E, D, mh, 5)
    layout = torch.tensor([[[1, 0], [1, 1]]])
    out, ln = osbb.sbblocksparse_attention(q, k, v, P, layout, block)
    t = 1 / math.sqrt(E)
    m = 2 * mh
    for i in (0, 7, 16, 31):
        num = torch.zeros(D, dtype=torch.float64)
        den = 0.0
        for j in range(S):
            if layout[0, i // block, j // block]:
                w = math.exp(t * float(q[0, i, 0] @ k[0, j, 0]))
            else:
                w = 0.0
                for r in range(mh):
                    a = math.sqrt(t) * float(P[r] @ q[0, i, 0])
                    b = math.sqrt(t) * float(P[r] @ k[0, j, 0])
                    w += math.exp(a + b) + math.exp(-a - b)
                w *= math.exp(-t / 2 * float(q[0, i, 0] @ q[0, i, 0]) - t / 2 * float(k[0, j, 0] @ k[0, j, 0])) / m
            num += w * v[0, j, 0]
            den += w
        assert torch.allclose(out[0, i, 0], num / den, rtol=1e-10, atol=1e-12)
        assert abs(float(ln[0, 0, i, 0]) - math.log(den)) < 1e-10


def test_invariants():
    B, T, S, H, E, D, mh, block = 2, 64, 64, 2, 16, 8, 8, 16
    q, k, v, P = _inputs(B, T, S, H, E, D, mh, 9)
    # values of one give outputs of one, whatever the support
    layout = _layout(H, 4, 4, 3)
    out, _ = osbb.sbblocksparse_attention(q, k, torch.ones_like(v), P, layout, block)
    assert (out - 1).abs().max() < 1e-10
    # full support: plain softmax attention and its logsumexp, the features drop out
    full = torch.ones(H, 4, 4, dtype=torch.long)
    out, ln = osbb.sbblocksparse_attention(q, k, v, P, full, block)
    s = torch.einsum('bthe,bshe->bhts', q, k) / math.sqrt(E)
    ref = torch.einsum('bhts,bshd->bthd', torch.softmax(s, -1), v)
    assert rel_err(out, ref) < 1e-10
    assert rel_err(ln, torch.logsumexp(s, -1, keepdim=True)) < 1e-10


def test_product_feature_map_matches_oracle():
    """fly_amd's torch feature map (used by the block-sparse Scatterbrain layer) against the oracle's,
    which tests/test_oracle_sblocal.py pins by loops."""
    from fly_amd.feature_maps_sb import softmax_kernel
    g = torch.Generator().manual_seed(2)
    x = torch.randn(2, 3, 20, 16, generator=g)
    P = osb.gaussian_orthogonal_random_matrix(8, 16, generator=g)
    for is_query in (True, False):
        f, ls = softmax_kernel(x, projection_matrix=P, is_query=is_query, softmax_temp=0.3)
        rf, rls = osb.softmax_kernel(x, P, is_query, softmax_temp=0.3)
        assert torch.allclose(f, rf, rtol=1e-6, atol=1e-7) and torch.allclose(ls, rls, rtol=1e-6, atol=1e-7)
    lf, _ = softmax_kernel(x, projection_matrix=P, is_query=True, return_log=True)
    f, _ = softmax_kernel(x, projection_matrix=P, is_query=True)
    assert torch.allclose(lf.exp(), f, rtol=1e-6)
