"""Pins the Scatterbrain-local oracle (oracle/sblocal.py) with checks that do not retype its
formulas: brute-force loops, an independent float64 closed form, and invariants.  CPU only."""
import math

import pytest
import torch

from oracle import sblocal as osb


def _inputs(B, T, S, H, E, D, mh, seed, scale=None):
    g = torch.Generator().manual_seed(seed)
    scale = E ** -0.25 if scale is None else scale
    q = torch.randn(B, T, H, E, generator=g, dtype=torch.float64) * scale
    k = torch.randn(B, S, H, E, generator=g, dtype=torch.float64) * scale
    v = torch.randn(B, S, H, D, generator=g, dtype=torch.float64)
    P = osb.gaussian_orthogonal_random_matrix(mh, E, generator=g, dtype=torch.float64)
    return q, k, v, P


@pytest.mark.parametrize('nrows,ncols', [(64, 64), (128, 64), (36, 21), (13, 21)])
def test_projection_blocks_are_scaled_orthogonal(nrows, ncols):
    g = torch.Generator().manual_seed(1)
    P = osb.gaussian_orthogonal_random_matrix(nrows, ncols, generator=g, dtype=torch.float64)
    assert P.shape == (nrows, ncols)
    unit = P / P.norm(dim=1, keepdim=True)
    for r0 in range(0, nrows, ncols):                      # rows of one QR block are orthonormal
        blk = unit[r0:r0 + ncols]
        assert torch.allclose(blk @ blk.t(), torch.eye(blk.shape[0], dtype=torch.float64), atol=1e-10)
    # row norms follow chi(ncols): mean ~ sqrt(ncols - 1/2)
    assert abs(P.norm(dim=1).mean() - math.sqrt(ncols - 0.5)) < 0.25 * math.sqrt(ncols)
    P1 = osb.gaussian_orthogonal_random_matrix(nrows, ncols, scaling=1, generator=g, dtype=torch.float64)
    assert torch.allclose(P1.norm(dim=1), torch.full((nrows,), math.sqrt(ncols), dtype=torch.float64))
    with pytest.raises(ValueError):
        osb.gaussian_orthogonal_random_matrix(4, 4, scaling=2)


@pytest.mark.parametrize('t', [None, 1.0, 0.235])
def test_feature_map_closed_form(t):
    """feat_q . feat_k * exp(ls_q + ls_k) must equal the un-stabilised positive random feature
    product (1/m) sum_r [e^{w_r.(q~+k~)} + e^{-w_r.(q~+k~)}] e^{-(|q~|^2+|k~|^2)/2}, x~ = sqrt(t) x,
    evaluated here with explicit Python loops."""
    q, k, _, P = _inputs(1, 5, 6, 1, 7, 3, 4, seed=3, scale=0.7)
    temp = t if t is not None else 1 / math.sqrt(7)
    fq, lq = osb.softmax_kernel(q[0, :, 0], P, True, softmax_temp=t)
    fk, lk = osb.softmax_kernel(k[0, :, 0], P, False, softmax_temp=t)
    assert fq.shape == (5, 8) and fk.shape == (6, 8) and lq.shape == (5, 1) and lk.shape == (1, 1)
    assert float(fq.max()) <= 1.0 + 1e-12 and float(fk.max()) <= 1.0 + 1e-12     # stabilised
    m = 8
    for i in range(5):
        for j in range(6):
            qt, kt = math.sqrt(temp) * q[0, i, 0], math.sqrt(temp) * k[0, j, 0]
            acc = 0.0
            for r in range(4):
                z = float(P[r] @ (qt + kt))
                acc += math.exp(z) + math.exp(-z)
            want = acc / m * math.exp(-0.5 * float(qt @ qt + kt @ kt))
            got = float(fq[i] @ fk[j]) * math.exp(float(lq[i]) + float(lk))
            assert got == pytest.approx(want, rel=1e-10)


def test_feature_map_is_unbiased_for_exp_kernel():
    """E[phi(q).phi(k)] = exp(t q.k): with 30000 features the relative error is small
    (cf. tests/models/attention/test_sblocal_attention.py:90-97 of the reference)."""
    q, k, _, _ = _inputs(1, 8, 8, 1, 16, 4, 2, seed=5)
    g = torch.Generator().manual_seed(0)
    P = osb.gaussian_orthogonal_random_matrix(15000, 16, generator=g, dtype=torch.float64)
    fq, lq = osb.softmax_kernel(q[0, :, 0], P, True)
    fk, lk = osb.softmax_kernel(k[0, :, 0], P, False)
    est = (fq @ fk.t()) * torch.exp(lq + lk)
    exact = torch.exp((q[0, :, 0] @ k[0, :, 0].t()) / 4.0)
    assert ((est - exact) / exact).abs().mean() < 0.05


@pytest.mark.parametrize('lc', [1, 3, 4, 7, 28, 200])
def test_local_products_against_loops(lc):
    g = torch.Generator().manual_seed(lc)
    B, H, T, S, E, D = 2, 2, 11, 9, 5, 3
    Q = torch.randn(B, H, T, E, generator=g, dtype=torch.float64)
    K = torch.randn(B, H, S, E, generator=g, dtype=torch.float64)
    V = torch.randn(B, H, S, D, generator=g, dtype=torch.float64)
    lens = torch.tensor([9, 4])
    got = osb.local_dot_product(Q, K, None, lens, lc, chunk=4)
    want = torch.full((B, H, T, lc), -1e24, dtype=torch.float64)
    for b in range(B):
        for h in range(H):
            for i in range(T):
                for j in range(lc):
                    s = i - lc // 2 + j
                    if 0 <= s < int(lens[b]):
                        want[b, h, i, j] = Q[b, h, i] @ K[b, h, s]
    assert torch.allclose(got, want, rtol=1e-12, atol=1e-12)
    A = torch.randn(B, H, T, lc, generator=g, dtype=torch.float64)
    got = osb.local_weighted_average(A, V, chunk=4)
    want = torch.zeros(B, H, T, D, dtype=torch.float64)
    for b in range(B):
        for h in range(H):
            for i in range(T):
                for j in range(lc):
                    s = i - lc // 2 + j
                    if 0 <= s < S:
                        want[b, h, i] += A[b, h, i, j] * V[b, h, s]
    assert torch.allclose(got, want, rtol=1e-12, atol=1e-12)


def test_band_definition_even_and_odd_windows():
    """Even lc: [i - lc/2, i + lc/2); odd lc: symmetric (test_sblocal_attention.py:77-82)."""
    Q = torch.eye(6, dtype=torch.float64).view(1, 1, 6, 6)
    K = torch.eye(6, dtype=torch.float64).view(1, 1, 6, 6)
    lens = torch.tensor([6])
    d4 = osb.local_dot_product(Q, K, None, lens, 4)[0, 0]
    # query 3 sees keys 1,2,3,4 in slots 0..3; the self product (=1) sits in slot lc//2 = 2
    assert d4[3].tolist() == [0.0, 0.0, 1.0, 0.0]
    assert d4[0].tolist() == [-1e24, -1e24, 1.0, 0.0]          # keys -2, -1 do not exist
    assert d4[5].tolist() == [0.0, 0.0, 1.0, -1e24]            # key 6 does not exist
    d3 = osb.local_dot_product(Q, K, None, lens, 3)[0, 0]
    assert d3[3].tolist() == [0.0, 1.0, 0.0]                   # keys 2,3,4
    assert d3[5].tolist() == [0.0, 1.0, -1e24]


@pytest.mark.parametrize('lc,mh,t,lens', [
    (3, 36, None, None), (4, 13, 1.0, [39, 12, 20]), (28, 36, 0.235, [10, 39, 25]), (33, 13, None, [39, 9, 30]),
    (512, 8, None, None)])
def test_forward_matches_dense_closed_form(lc, mh, t, lens):
    """The reference op sequence (band-packed tensors, stabilisers, overlap subtraction) against the
    estimator written directly as a dense (T,S) matrix in float64."""
    q, k, v, P = _inputs(3, 47, 39, 2, 21, 17, mh, seed=2357, scale=0.6)
    lens = None if lens is None else torch.tensor(lens)
    out, ln = osb.sblocal_attention(q, k, v, P, lc, softmax_temp=t, key_lengths=lens)
    out2, ln2, A = osb.dense_closed_form(q, k, v, P, lc, softmax_temp=t, key_lengths=lens)
    assert out.shape == (3, 47, 2, 17) and ln.shape == (3, 2, 47, 1)
    assert torch.allclose(out, out2, rtol=1e-9, atol=1e-11)
    assert torch.allclose(ln, ln2, rtol=1e-9, atol=1e-11)
    # invariants of the reference's test: non-negative weights, exact values on the band
    assert bool((A >= 0).all())
    temp = t or 1 / math.sqrt(21)
    exact = torch.exp(temp * torch.einsum('bthe,bshe->bhts', q, k))
    i = torch.arange(47).view(47, 1)
    j = torch.arange(39).view(1, 39)
    band = ((j - i) >= -(lc // 2)) & ((j - i) < (lc + 1) // 2)
    if lens is not None:
        band = band.view(1, 1, 47, 39) & (j.view(1, 1, 1, 39) < lens.view(3, 1, 1, 1))
    else:
        band = band.view(1, 1, 47, 39).expand(3, 2, 47, 39)
    band = band.expand(3, 2, 47, 39)
    assert torch.allclose(A[band], exact[band], rtol=1e-12)


def test_value_of_ones_gives_ones_and_wide_band_is_full_attention():
    q, k, v, P = _inputs(2, 40, 40, 2, 16, 8, 6, seed=11)
    out, _ = osb.sblocal_attention(q, k, torch.ones_like(v), P, 9, key_lengths=torch.tensor([40, 17]))
    assert torch.allclose(out, torch.ones_like(out), atol=1e-12)
    out, ln = osb.sblocal_attention(q, k, v, P, 200)
    att = torch.softmax(torch.einsum('bthe,bshe->bhts', q, k) / 4.0, dim=-1)
    full = torch.einsum('bhts,bshd->bthd', att, v)
    assert torch.allclose(out, full, atol=1e-10)
    lse = torch.logsumexp(torch.einsum('bthe,bshe->bhts', q, k) / 4.0, dim=-1, keepdim=True)
    assert torch.allclose(ln, lse, atol=1e-10)


def test_float32_oracle_is_close_to_float64():
    q, k, v, P = _inputs(2, 300, 300, 1, 64, 64, 64, seed=0)
    o64, l64 = osb.sblocal_attention(q, k, v, P, 128)
    o32, l32 = osb.sblocal_attention(q.float(), k.float(), v.float(), P.float(), 128)
    assert float((o32.double() - o64).abs().max() / o64.abs().max()) < 1e-5
    assert float((l32.double() - l64).abs().max() / l64.abs().max()) < 1e-5


def test_local_attention_equals_dense_masked_softmax():
    """LocalAttention restated from the band-packed op sequence against a dense softmax over the same
    support (a different route: -inf mask on the full (T,S) matrix), with key lengths and T != S."""
    g = torch.Generator().manual_seed(8)
    for (B, T, S, H, E, D, lc, lens) in [(2, 40, 40, 2, 8, 5, 7, None), (2, 33, 50, 1, 4, 6, 12, [50, 21]),
                                         (1, 50, 20, 2, 4, 4, 9, [13])]:
        q = torch.randn(B, T, H, E, generator=g, dtype=torch.float64)
        k = torch.randn(B, S, H, E, generator=g, dtype=torch.float64)
        v = torch.randn(B, S, H, D, generator=g, dtype=torch.float64)
        kl = None if lens is None else torch.tensor(lens)
        out = osb.local_attention(q, k, v, lc, softmax_temp=0.4, key_lengths=kl)
        i = torch.arange(T).view(T, 1)
        j = torch.arange(S).view(1, S)
        band = ((j - i) >= -(lc // 2)) & ((j - i) < (lc + 1) // 2)
        limit = torch.full((B,), S) if kl is None else kl
        ok = band.view(1, 1, T, S) & (j.view(1, 1, 1, S) < limit.view(B, 1, 1, 1))
        s = 0.4 * torch.einsum('bthe,bshe->bhts', q, k)
        w = torch.softmax(s.masked_fill(~ok, float('-inf')), dim=-1)
        w = torch.where(ok.any(-1, keepdim=True), w, torch.zeros_like(w))      # rows without a valid key
        ref = torch.einsum('bhts,bshd->bthd', w, v)
        assert (out - ref).abs().max() < 1e-12


def test_local_attention_with_an_additive_mask():
    """LocalAttention with attn_mask (local_attention.py:53-56, 68-81: additive_matrix_finite added to Q K^T inside
    the band-packed product).  Rows that keep a visible key equal a dense softmax with -inf on band, lengths and mask;
    a row whose visible keys are all masked has equal scores everywhere in its packed band, i.e. weights
    1 / local_context, and its output is the sum of its visible values over local_context (the reference leaves such
    rows as they are, :76-81); a general finite bias equals the dense softmax of t (q.k + bias)."""
    g = torch.Generator().manual_seed(18)
    for (B, T, S, H, E, D, lc, lens) in [(2, 40, 40, 2, 8, 5, 7, None), (2, 33, 50, 1, 4, 6, 12, [50, 21])]:
        q = torch.randn(B, T, H, E, generator=g, dtype=torch.float64)
        k = torch.randn(B, S, H, E, generator=g, dtype=torch.float64)
        v = torch.randn(B, S, H, D, generator=g, dtype=torch.float64)
        kl = None if lens is None else torch.tensor(lens)
        keep = torch.rand(T, S, generator=g) < 0.6
        keep[3] = False                                     # a query with every key hidden
        keep[T - 2] = False
        add = (~keep).double() * -1e24
        out = osb.local_attention(q, k, v, lc, softmax_temp=0.4, key_lengths=kl, attn_mask_additive=add)
        i = torch.arange(T).view(T, 1)
        j = torch.arange(S).view(1, S)
        band = ((j - i) >= -(lc // 2)) & ((j - i) < (lc + 1) // 2)
        limit = torch.full((B,), S) if kl is None else kl
        vis = band.view(1, 1, T, S) & (j.view(1, 1, 1, S) < limit.view(B, 1, 1, 1))
        ok = vis & keep.view(1, 1, T, S)
        s = 0.4 * torch.einsum('bthe,bshe->bhts', q, k)
        w = torch.softmax(s.masked_fill(~ok, float('-inf')), dim=-1).nan_to_num(0.0)
        hidden_row = vis.any(-1, keepdim=True) & ~ok.any(-1, keepdim=True)
        w = torch.where(hidden_row, vis.double() / lc, w)
        ref = torch.einsum('bhts,bshd->bthd', w, v)
        assert bool(hidden_row.any()) and (out - ref).abs().max() < 1e-12
        bias = torch.randn(T, S, generator=g, dtype=torch.float64)
        out = osb.local_attention(q, k, v, lc, softmax_temp=0.4, key_lengths=kl, attn_mask_additive=bias)
        w = torch.softmax((0.4 * (torch.einsum('bthe,bshe->bhts', q, k) + bias)).masked_fill(~vis, float('-inf')), -1)
        ref = torch.einsum('bhts,bshd->bthd', w.nan_to_num(0.0), v)
        assert (out - ref).abs().max() < 1e-12


@pytest.mark.parametrize('B,T,S,H,E,D,mh,lc,lens', [(1, 40, 40, 2, 16, 16, 8, 12, None),
                                                    (2, 70, 55, 2, 16, 24, 8, 13, [55, 31]),
                                                    (1, 300, 300, 1, 8, 8, 4, 64, None)])
def test_written_out_backward_matches_autograd_through_the_oracle(B, T, S, H, E, D, mh, lc, lens):
    """fly_amd.sblocal_backward (the gradients written out: band terms plus global low-rank terms plus
    the feature-map chain rule) against autograd through the oracle's op sequence, in float64, with
    chunks smaller than the sequence, T != S, an odd window and key lengths."""
    from fly_amd.sblocal_backward import sblocal_backward
    g = torch.Generator().manual_seed(0)
    q = (torch.randn(B, T, H, E, generator=g).double() * 0.7).requires_grad_()
    k = (torch.randn(B, S, H, E, generator=g).double() * 0.7).requires_grad_()
    v = torch.randn(B, S, H, D, generator=g).double().requires_grad_()
    P = osb.gaussian_orthogonal_random_matrix(mh, E, generator=g, dtype=torch.float64)
    kl = None if lens is None else torch.tensor(lens)
    out, ln = osb.sblocal_attention(q, k, v, P, lc, key_lengths=kl)
    w = torch.randn(out.shape, generator=g).double()
    (out * w).sum().backward()
    dq, dk, dv = sblocal_backward(q.detach(), k.detach(), v.detach(), P, lc, None, kl, out.detach(), ln.detach(), w,
                                  chunk=32)
    for got, ref in ((dq, q.grad), (dk, k.grad), (dv, v.grad)):
        assert float((got - ref).abs().max() / ref.abs().max()) < 1e-10
    # chunks taken one group at a time give the same sums
    again = sblocal_backward(q.detach(), k.detach(), v.detach(), P, lc, None, kl, out.detach(), ln.detach(), w,
                             chunk=32, max_elements=1)
    for got, ref in zip(again, (dq, dk, dv)):
        assert float((got - ref).abs().max()) < 1e-12
    if lens is not None:
        assert float(dk[1, lens[1]:].abs().max()) == 0.0 and float(dv[1, lens[1]:].abs().max()) == 0.0


@pytest.mark.parametrize('B,T,S,H,E,D,lc,lens', [(1, 40, 40, 2, 16, 16, 12, None), (2, 70, 55, 2, 16, 24, 13, [55, 31]),
                                                 (1, 300, 300, 1, 8, 8, 64, None)])
def test_local_backward_matches_autograd_through_the_oracle(B, T, S, H, E, D, lc, lens):
    """fly_amd.local_backward (band softmax evaluated again per chunk of queries) against autograd
    through the oracle's LocalAttention op sequence, in float64, with chunks smaller than the
    sequence, T != S, an odd window and key lengths (queries past every visible key included)."""
    from fly_amd.local_attention import local_backward
    g = torch.Generator().manual_seed(1)
    q = torch.randn(B, T, H, E, generator=g).double().requires_grad_()
    k = torch.randn(B, S, H, E, generator=g).double().requires_grad_()
    v = torch.randn(B, S, H, D, generator=g).double().requires_grad_()
    kl = None if lens is None else torch.tensor(lens)
    out = osb.local_attention(q, k, v, lc, key_lengths=kl)
    w = torch.randn(out.shape, generator=g).double()
    (out * w).sum().backward()
    dq, dk, dv = local_backward(q.detach(), k.detach(), v.detach(), lc, None, kl, w, chunk=32)
    for got, ref in ((dq, q.grad), (dk, k.grad), (dv, v.grad)):
        assert float((got - ref).abs().max() / ref.abs().max()) < 1e-10
    again = local_backward(q.detach(), k.detach(), v.detach(), lc, None, kl, w, chunk=32, max_elements=1)
    for got, ref in zip(again, (dq, dk, dv)):
        assert float((got - ref).abs().max()) < 1e-12
    if lens is not None:
        assert float(dk[1, lens[1]:].abs().max()) == 0.0 and float(dv[1, lens[1]:].abs().max()) == 0.0


def test_dropout_multiplier_of_the_oracle_and_the_restated_hash():
    """dropout_multiplier multiplies exp(QK - log_normalization) and nothing else (sblocal_attention.py:116-119):
    with an all-ones multiplier the oracle is unchanged, with zeros only the low-rank part remains, the normaliser never
    moves; a multiplier that drops one pair removes exactly that pair's exact weight times its value.  The restated
    hash of the kernels: keeps with probability 1 - p, independent of one another to what a chi-square on pairs of
    neighbours can see, scaled by 1 / (1 - p), all kept at p = 0, different for different seeds."""
    g = torch.Generator().manual_seed(0)
    B, T, S, H, E, D, lc = 2, 20, 17, 2, 8, 5, 6
    q, k, v = (torch.randn(B, n, H, c, generator=g, dtype=torch.float64) * 0.5 for n, c in ((T, E), (S, E), (S, D)))
    P = osb.gaussian_orthogonal_random_matrix(6, E, generator=g, dtype=torch.float64)
    out, ln = osb.sblocal_attention(q, k, v, P, lc)
    ones = torch.ones(B, H, T, S, dtype=torch.float64)
    out1, ln1 = osb.sblocal_attention(q, k, v, P, lc, dropout_multiplier=ones)
    assert torch.equal(out1, out) and torch.equal(ln1, ln)
    one_gone = ones.clone()
    b, h, i, s = 1, 0, 9, 10                                   # inside the band of query 9: keys 6 .. 11
    one_gone[b, h, i, s] = 0
    out2, ln2 = osb.sblocal_attention(q, k, v, P, lc, dropout_multiplier=one_gone)
    t = 1 / math.sqrt(E)
    weight = torch.exp(t * (q[b, i, h] @ k[b, s, h]) - ln[b, h, i, 0])
    diff = out - out2
    assert torch.equal(ln2, ln)
    assert torch.allclose(diff[b, i, h], weight * v[b, s, h], rtol=1e-12, atol=1e-15)
    diff[b, i, h] = 0
    assert float(diff.abs().max()) == 0.0
    far = ones.clone()
    far[b, h, i, 0] = 0                                        # outside the band: no exact weight there, nothing changes
    assert torch.equal(osb.sblocal_attention(q, k, v, P, lc, dropout_multiplier=far)[0], out)

    for p in (0.1, 0.5, 0.9):
        keep = osb.dropout_keep(2024, p, 2, 3, 300, 257)
        kept = keep > 0
        assert abs(float(kept.double().mean()) - (1 - p)) < 4 * math.sqrt(p * (1 - p) / kept.numel()) + 1e-4
        realised = int(p * 65536) / 65536                      # the threshold has 16 bits; the scale is that of the realised p
        assert abs(realised - p) < 2 ** -16
        assert torch.equal(keep[kept].unique(), torch.tensor([1 / (1 - realised)], dtype=torch.float64))
        # neighbouring keys and neighbouring queries: joint keep frequency = (1 - p)^2 within sampling error
        for a_, b_ in ((kept[..., :-1], kept[..., 1:]), (kept[..., :-1, :], kept[..., 1:, :])):
            joint = float((a_ & b_).double().mean())
            assert abs(joint - (1 - p) ** 2) < 5 * math.sqrt((1 - p) ** 2 / a_.numel()) + 2e-3, (p, joint)
    assert bool((osb.dropout_keep(7, 0.0, 1, 1, 10, 10) == 1).all())
    assert not torch.equal(osb.dropout_keep(7, 0.5, 1, 2, 64, 64), osb.dropout_keep(8, 0.5, 1, 2, 64, 64))
    assert not torch.equal(osb.dropout_keep(7, 0.5, 1, 2, 64, 64), osb.dropout_keep(7 + (1 << 40), 0.5, 1, 2, 64, 64))
