"""Pins the block-sparse oracle (oracle/blocksparse.py): storage format against per-block loops,
matmuls / row ops against dense torch ops on densified operands, layouts against the closed form
and the known block counts, look-up tables against brute-force enumeration.  CPU only."""
import math

import pytest
import torch

from oracle import blocksparse as ob


def _layout(H, p, r, seed, density=0.5):
    g = torch.Generator().manual_seed(seed)
    return (torch.rand(H, p, r, generator=g) < density).long()


def test_format_helpers_against_loops():
    H, p, r, blk, blk1 = 2, 3, 4, 4, 2
    layout = _layout(H, p, r, 0)
    g = torch.Generator().manual_seed(1)
    x = torch.randn(5, H, p * blk, r * blk1, generator=g)
    sp = ob.sparsify_tensor(x, layout)
    n = 0
    for h in range(H):
        for i in range(p):
            for j in range(r):
                if layout[h, i, j]:
                    assert torch.equal(sp[:, n], x[:, h, i * blk:(i + 1) * blk, j * blk1:(j + 1) * blk1])
                    n += 1
    assert sp.shape == (5, n, blk, blk1)
    dense = ob.densify_tensor(sp, layout, value=-7.0)
    masked = ob.mask_tensor(x, layout, value=-7.0)
    assert torch.equal(dense, masked)
    keep = layout.bool().repeat_interleave(blk, 1).repeat_interleave(blk1, 2)
    assert torch.equal(masked[:, keep], x[:, keep]) and bool((masked[:, ~keep] == -7.0).all())
    rows = torch.randn(5, H, p * blk, generator=g)
    bc = ob.sparsify_broadcast_tensor(rows, layout, blk)
    nz = layout.nonzero()
    for n, (h, i, j) in enumerate(nz.tolist()):
        assert torch.equal(bc[:, n, :, 0], rows[:, h, i * blk:(i + 1) * blk])


@pytest.mark.parametrize('trans_a,trans_b', [(False, False), (True, False), (False, True), (True, True)])
def test_matmuls_against_dense(trans_a, trans_b):
    H, p, r, blk, Z = 2, 3, 4, 8, 2
    layout = _layout(H, p, r, 2)
    g = torch.Generator().manual_seed(3)
    nnz = int(layout.sum())
    K = 16
    a = torch.randn((Z, H, K, p * blk) if trans_a else (Z, H, p * blk, K), generator=g, dtype=torch.float64)
    b = torch.randn((Z, H, r * blk, K) if trans_b else (Z, H, K, r * blk), generator=g, dtype=torch.float64)
    A = a.transpose(-1, -2) if trans_a else a
    Bm = b.transpose(-1, -2) if trans_b else b
    full = A @ Bm
    c = ob.sdd(a, b, layout, blk, trans_a, trans_b)
    for n, (h, i, j) in enumerate(layout.nonzero().tolist()):
        assert torch.allclose(c[:, n], full[:, h, i * blk:(i + 1) * blk, j * blk:(j + 1) * blk])
    sp = torch.randn(Z, nnz, blk, blk, generator=g, dtype=torch.float64)
    spd = torch.zeros(Z, H, p * blk, r * blk, dtype=torch.float64)
    for n, (h, i, j) in enumerate(layout.nonzero().tolist()):
        spd[:, h, i * blk:(i + 1) * blk, j * blk:(j + 1) * blk] = sp[:, n]
    inner = (p if trans_a else r) * blk
    d = torch.randn((Z, H, 5, inner) if trans_b else (Z, H, inner, 5), generator=g, dtype=torch.float64)
    want = (spd.transpose(-1, -2) if trans_a else spd) @ (d.transpose(-1, -2) if trans_b else d)
    assert torch.allclose(ob.dsd(sp, d, layout, blk, trans_a, trans_b), want)
    inner = (r if trans_b else p) * blk
    d = torch.randn((Z, H, inner, 5) if trans_a else (Z, H, 5, inner), generator=g, dtype=torch.float64)
    want = (d.transpose(-1, -2) if trans_a else d) @ (spd.transpose(-1, -2) if trans_b else spd)
    assert torch.allclose(ob.dds(d, sp, layout, blk, trans_a, trans_b), want)


def test_block_softmax_and_reductions_against_dense():
    """What tests/models/attention/test_blocksparse_attention.py:69-80 of the reference asserts."""
    H, p, r, blk, Z = 3, 4, 3, 4, 2
    layout = _layout(H, p, r, 4)
    layout[1, 2, :] = 0
    g = torch.Generator().manual_seed(5)
    nnz = int(layout.sum())
    x = torch.randn(Z, nnz, blk, blk, generator=g)
    dense = ob.densify_tensor(x, layout, value=float('-inf'))
    want = torch.softmax(dense * 0.23, dim=-1)
    zero_rows = (~layout.bool()).all(-1, keepdim=True).repeat_interleave(blk, 1)
    want = want.masked_fill(zero_rows, 0.0)
    got = ob.densify_tensor(ob.block_softmax(x, layout, blk, scale=0.23), layout)
    assert torch.allclose(got, want, atol=1e-7)
    # additive / multiplicative masks
    kpm_bool = torch.rand(Z, r * blk, generator=g) < 0.7
    am_bool = torch.rand(p * blk, r * blk, generator=g) < 0.7
    want = torch.softmax(dense + torch.log(kpm_bool.float())[:, None, None] + torch.log(am_bool.float()), -1)
    got = ob.block_softmax(x, layout, blk, key_padding_mask=torch.log(kpm_bool.float()), attn_mask=am_bool.float(),
                           attn_mask_mode='mul')
    got = ob.densify_tensor(got, layout)
    keep = layout.bool().repeat_interleave(blk, 1).repeat_interleave(blk, 2).expand(Z, -1, -1, -1)
    assert torch.equal(got[keep].isnan(), want[keep].isnan())
    assert torch.allclose(got[keep].nan_to_num(), want[keep].nan_to_num(), atol=1e-7)
    lse = torch.logsumexp(dense, -1).masked_fill(zero_rows.squeeze(-1), 0.0)
    assert torch.allclose(ob.block_logsumexp(x, layout, blk), lse, atol=1e-6)
    assert torch.allclose(ob.block_sum(x, layout, blk), ob.densify_tensor(x, layout).sum(-1), atol=1e-6)


def test_butterfly_factor_known_matrices():
    """n = 4, twiddle = 1..8: factor 0 couples neighbours (stride 1), factor 1 couples i and i^2; the
    expected matrices follow from the definition in src/ops/butterfly_factor.py:8-26."""
    tw = torch.arange(1, 9, dtype=torch.float32).reshape(2, 2, 2)
    f0 = ob.butterfly_factor_to_matrix(tw, 0)
    assert f0.tolist() == [[1, 2, 0, 0], [3, 4, 0, 0], [0, 0, 5, 6], [0, 0, 7, 8]]
    f1 = ob.butterfly_factor_to_matrix(tw, 1)
    assert f1.tolist() == [[1, 0, 2, 0], [0, 5, 0, 6], [3, 0, 4, 0], [0, 7, 0, 8]]


@pytest.mark.parametrize('bs,nf', [(8, 2), (16, 2), (8, 3), (4, 1), (32, 5)])
def test_flat_butterfly_pattern_closed_form(bs, nf):
    lay = ob.flat_butterfly_layout(bs, bs, bs, nf, block=1)
    for i in range(bs):
        for j in range(bs):
            want = (i == j) or any(j == (i ^ (1 << k)) for k in range(nf))
            assert int(lay[i, j]) == int(want)


def test_layout_block_counts_of_the_baseline_configs():
    fc1 = ob.flat_butterfly_layout(3072, 768, 8, 2, 32)
    fc2 = ob.flat_butterfly_layout(768, 3072, 8, 2, 32)
    assert fc1.shape == (96, 24) and fc2.shape == (24, 96) and fc1.dtype == torch.int32
    assert int(fc1.sum()) == 864 and int(fc2.sum()) == 864                       # density 3/8
    att = ob.flat_butterfly_layout(4096, 4096, 8, 2, 32)
    assert att.shape == (128, 128) and int(att.sum()) == 6144
    both = ((att + ob.band_layout(128, 128, 4)) > 0)
    assert int(both.sum()) == 6204
    row_nnz = both.sum(-1)
    assert int(row_nnz.min()) == 48 and int(row_nnz.max()) == 52
    # global rows / columns and the shuffle option
    glob = ob.flat_butterfly_layout(256, 256, 8, 1, 32, global_size=32)
    assert bool(glob[0].all()) and bool(glob[:, 0].all())
    sh = ob.flat_butterfly_layout(256, 256, 8, 2, 32, shuffle=True)
    assert int(sh.sum()) == int(ob.flat_butterfly_layout(256, 256, 8, 2, 32).sum())


def test_lookup_tables_by_enumeration():
    layout = _layout(3, 4, 5, 7)
    layout[2, 1, :] = 0
    lut = ob.sdd_lut(layout)
    want = [(h, i, j) for h in range(3) for i in range(4) for j in range(5) if layout[h, i, j]]
    assert lut.dtype == torch.int32 and lut[:, :3].tolist() == [list(x) for x in want]
    assert lut[:, 3].tolist() == list(range(len(want)))
    rl, max_nnz, n_head, n_row = ob.row_lut(layout, 16)
    sizes = layout.sum(-1).flatten()
    assert (max_nnz, n_head, n_row) == (int(sizes.max()), 3, 64)
    n_seg = 12
    hdr = rl[:2 * n_seg].view(n_seg, 2)
    assert hdr[:, 0].tolist() == sizes.tolist()
    off = 0
    for s in range(n_seg):
        assert int(hdr[s, 1]) == 2 * n_seg + 4 * off
        off += int(sizes[s])
    core = rl[2 * n_seg:].view(-1, 4)
    assert core[:, 0].tolist() == list(range(len(want)))
    assert core[:, 1:].tolist() == [[j, i, h] for (h, i, j) in want]
    for by_rows in (True, False):
        ptr, blk, inner = ob.segment_table(layout, by_rows)
        ids = {x: n for n, x in enumerate(want)}
        k = 0
        for h in range(3):
            for o in range(4 if by_rows else 5):
                items = [(ids[(h, o, x)], x) for x in range(5) if layout[h, o, x]] if by_rows else \
                        [(ids[(h, x, o)], x) for x in range(4) if layout[h, x, o]]
                seg = h * (4 if by_rows else 5) + o
                assert int(ptr[seg]) == k
                assert list(zip(blk[k:k + len(items)].tolist(), inner[k:k + len(items)].tolist())) == items
                k += len(items)
        assert int(ptr[-1]) == k == len(want)


def test_attention_and_linear_compositions():
    g = torch.Generator().manual_seed(9)
    B, T, S, H, E, D, blk = 2, 40, 36, 2, 12, 20, 16
    q = torch.randn(B, T, H, E, generator=g)
    k = torch.randn(B, S, H, E, generator=g)
    v = torch.randn(B, S, H, D, generator=g)
    master = torch.ones(H, 4, 4, dtype=torch.long)            # dense layout: must equal full attention
    lens = torch.tensor([36, 20])
    out = ob.blocksparse_attention(q, k, v, master, blk, key_lengths=lens)
    s = torch.einsum('bthe,bshe->bhts', q, k) / math.sqrt(E)
    s = s.masked_fill(~(torch.arange(S).view(1, 1, 1, S) < lens.view(B, 1, 1, 1)), float('-inf'))
    want = torch.einsum('bhts,bshd->bthd', torch.softmax(s, -1), v)
    assert out.shape == (B, T, H, D) and torch.allclose(out, want, atol=1e-5)
    layout = ob.flat_butterfly_layout(64, 96, 2, 1, 32)
    W = torch.randn(int(layout.sum()), 32, 32, generator=g)
    x = torch.randn(7, 90, generator=g)
    dense = ob.densify_tensor(W.unsqueeze(0), layout.unsqueeze(0))[0, 0]
    y = ob.blocksparse_linear(x, W, layout, 32, out_features=50)
    assert torch.allclose(y, (torch.nn.functional.pad(x, (0, 6)) @ dense.t())[:, :50], atol=1e-5)
