"""Parity of the HIP block-sparse matmuls / row ops against the CPU oracle (GPU box only)."""
import math

import pytest
import torch

from conftest import rel_err
from oracle import blocksparse as ob

pytestmark = pytest.mark.gpu
DEV = 'cuda:0'
TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2, torch.float16: 2e-3}


def random_layout(H, p, r, seed, density=0.5):
    g = torch.Generator().manual_seed(seed)
    return (torch.rand(H, p, r, generator=g) < density).long()


@pytest.mark.parametrize('dtype', [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize('block', [16, 32, 64, 128])
def test_sdd_softmax_dsd_pipeline(block, dtype):
    """The reference's own pipeline test (tests/models/attention/test_blocksparse_attention.py:32-81)
    at several block sizes and dtypes."""
    from fly_amd import matmul, softmax
    print('case', block, dtype, flush=True)
    Z, H, p, r, K = 2, 3, 4, 3, 48 if block == 16 else 64
    g = torch.Generator().manual_seed(2357)
    q = torch.randn(Z, H, p * block, K, generator=g).to(dtype)
    k = torch.randn(Z, H, r * block, K, generator=g).to(dtype)
    v = torch.randn(Z, H, r * block, K, generator=g).to(dtype)
    layout = random_layout(H, p, r, 1)
    layout[0, 1, :] = 0                                  # an empty block-row
    tol = TOL[dtype]

    qk = matmul(layout, block, 'sdd', trans_a=False, trans_b=True)(q.to(DEV), k.to(DEV))
    qk_ref = ob.sdd(q, k, layout, block, trans_b=True)
    assert qk.shape == qk_ref.shape
    assert rel_err(qk, qk_ref) <= tol

    attn = softmax(layout, block)(qk.clone(), scale=0.23)
    attn_ref = ob.block_softmax(qk.cpu(), layout, block, scale=0.23)
    assert rel_err(attn, attn_ref) <= tol

    out = matmul(layout, block, 'dsd')(attn, v.to(DEV))
    out_ref = ob.dsd(attn.cpu(), v, layout, block)
    assert rel_err(out, out_ref) <= tol
    assert out.shape == (Z, H, p * block, K)
    # rows of the empty block-row are exactly zero
    assert float(out[:, 0, block:2 * block].abs().max()) == 0.0


@pytest.mark.parametrize('trans_a,trans_b', [(False, False), (True, False), (False, True), (True, True)])
@pytest.mark.parametrize('mode', ['sdd', 'dsd', 'dds'])
def test_matmul_modes_and_transposes(mode, trans_a, trans_b):
    from fly_amd import matmul
    print('case', mode, trans_a, trans_b, flush=True)
    block, Z, H, p, r = 32, 2, 2, 3, 5
    layout = random_layout(H, p, r, 3)
    g = torch.Generator().manual_seed(11)
    nnz = int(layout.sum())
    if mode == 'sdd':
        K = 48
        a = torch.randn((Z, H, K, p * block) if trans_a else (Z, H, p * block, K), generator=g)
        b = torch.randn((Z, H, r * block, K) if trans_b else (Z, H, K, r * block), generator=g)
        ref = ob.sdd(a, b, layout, block, trans_a, trans_b)
    elif mode == 'dsd':
        a = torch.randn(Z, nnz, block, block, generator=g)
        inner = (p if trans_a else r) * block
        N = 40
        b = torch.randn((Z, H, N, inner) if trans_b else (Z, H, inner, N), generator=g)
        ref = ob.dsd(a, b, layout, block, trans_a, trans_b)
    else:
        b = torch.randn(Z, nnz, block, block, generator=g)
        inner = (r if trans_b else p) * block
        M = 72
        a = torch.randn((Z, H, inner, M) if trans_a else (Z, H, M, inner), generator=g)
        ref = ob.dds(a, b, layout, block, trans_a, trans_b)
    out = matmul(layout, block, mode, trans_a=trans_a, trans_b=trans_b)(a.to(DEV), b.to(DEV))
    assert out.shape == ref.shape
    assert rel_err(out, ref) <= 1e-5


def test_softmax_masks_and_rowreduce():
    from fly_amd import softmax, logsumexp, blocksparse_sum
    block, Z, H, p, r = 32, 3, 2, 4, 6
    layout = random_layout(H, p, r, 5, density=0.6)
    layout[1, 2, :] = 0
    g = torch.Generator().manual_seed(4)
    nnz = int(layout.sum())
    x = torch.randn(Z, nnz, block, block, generator=g)
    lens = torch.tensor([r * block, 70, 1])
    kpm = torch.log((torch.arange(r * block).view(1, -1) < lens.view(-1, 1)).float())
    am_bool = torch.rand(p * block, r * block, generator=g) < 0.7
    am = torch.log(am_bool.float())
    for kw_dev, kw_ref in [
        (dict(key_padding_mask=kpm.to(DEV)), dict(key_padding_mask=kpm)),
        (dict(attn_mask=am.to(DEV)), dict(attn_mask=am)),
        (dict(key_padding_mask=kpm.to(DEV), attn_mask=am.to(DEV)), dict(key_padding_mask=kpm, attn_mask=am)),
        (dict(attn_mask=am_bool.float().to(DEV), attn_mask_mode='mul'),
         dict(attn_mask=am_bool.float(), attn_mask_mode='mul')),
    ]:
        got = softmax(layout, block)(x.clone().to(DEV), scale=0.5, **kw_dev).cpu()
        ref = ob.block_softmax(x, layout, block, scale=0.5, **kw_ref)
        assert torch.equal(got.isnan(), ref.isnan())
        assert rel_err(got.nan_to_num(), ref.nan_to_num()) <= 1e-5
    assert rel_err(logsumexp(layout, block)(x.to(DEV)), ob.block_logsumexp(x, layout, block)) <= 1e-5
    assert rel_err(blocksparse_sum(layout, block)(x.to(DEV)), ob.block_sum(x, layout, block)) <= 1e-5
    # long rows take the multi-pass kernel
    layout = torch.ones(1, 1, 80, dtype=torch.long)
    x = torch.randn(2, 80, 32, 32, generator=g)
    got = softmax(layout, 32)(x.clone().to(DEV), scale=1.3).cpu()
    assert rel_err(got, ob.block_softmax(x, layout, 32, scale=1.3)) <= 1e-5


def test_blocksparse_attention_module():
    """BlockSparseAttention end to end with masks and sizes that need padding
    (cf. tests/models/attention/test_blocksparse_attention.py:83-142)."""
    from fly_amd import BlockSparseAttention, FullMask, LengthMask

    class Cfg:
        block = 16

        def make_layout(self, seqlen):
            nb = seqlen // self.block
            lay = ob.band_layout(nb, nb, 1)
            lay[:, 0] = 1
            return lay.unsqueeze(0).repeat(3, 1, 1)

    B, T, S, H, E, D = 2, 235, 179, 3, 15, 33
    g = torch.Generator().manual_seed(0)
    q = torch.randn(B, T, H, E, generator=g)
    k = torch.randn(B, S, H, E, generator=g)
    v = torch.randn(B, S, H, D, generator=g)
    lengths = torch.tensor([S, 77])
    am_bool = torch.rand(T, S, generator=g) < 0.8
    mod = BlockSparseAttention(Cfg(), attention_dropout=0.0, max_seq_length=256).to(DEV)
    out, _ = mod(q.to(DEV), k.to(DEV), v.to(DEV), attn_mask=FullMask(am_bool.to(DEV)),
                 key_padding_mask=LengthMask(lengths.to(DEV), max_len=S))
    ref = ob.blocksparse_attention(q, k, v, mod.master_layout.cpu(), 16, key_lengths=lengths,
                                   attn_mask_bool=am_bool)
    assert out.shape == (B, T, H, D)
    assert rel_err(out, ref) <= 1e-5


def test_blocksparse_linear_and_sparse_lr():
    """Pixelfly linear at small, non-aligned sizes (cf. tests/models/layers/test_blocksparse_linear.py:88-134)."""
    from fly_amd import BlockSparseLinear, FlatBlockButterflySparsityConfig, SparseLRLinear
    torch.manual_seed(0)
    cfg = FlatBlockButterflySparsityConfig(8, 2, block=32)
    lin = BlockSparseLinear(497, 698, cfg).to(DEV)
    x = torch.randn(3, 57, 497)
    y = lin(x.to(DEV))
    ref = ob.blocksparse_linear(x, lin.weight.detach().cpu(), lin.layout.cpu(), 32, lin.bias.detach().cpu(), 698)
    assert y.shape == (3, 57, 698)
    assert rel_err(y, ref) <= 1e-5

    slr = SparseLRLinear(256, 512, {'_target_': 'src.models.layers.blocksparse_linear.BlockSparseLinear',
                                    'sparsity_config': cfg}, rank=16).to(DEV)
    x = torch.randn(100, 256)
    y = slr(x.to(DEV))
    sp = ob.blocksparse_linear(x, slr.sparse.weight.detach().cpu(), slr.sparse.layout.cpu(), 32, None, 512)
    ref = ob.sparse_lr_linear(x, sp, slr.low_rank.lr_weight1.detach().cpu(), slr.low_rank.lr_weight2.detach().cpu(),
                              slr.gate.weight.detach().cpu(), slr.gate.bias.detach().cpu(), slr.bias.detach().cpu())
    assert rel_err(y, ref) <= 1e-4


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16])
@pytest.mark.parametrize('p,r,K,N', [(8, 6, 64, 64), (7, 5, 32, 40), (9, 4, 128, 136), (2, 3, 96, 72)])
def test_shared_tile_kernels(p, r, K, N, dtype, monkeypatch):
    """The SDD / DSD kernels that share tiles among four block-rows (32x32 blocks, 2-byte types),
    forced on for layouts with and without common columns: ragged last group, an empty group, an
    empty row inside a group, reduction sizes 32..128, dense widths that are not multiples of 64."""
    from fly_amd import matmul
    import fly_amd.blocksparse_matmul as bm
    monkeypatch.setattr(bm, 'UNION_MIN_SHARING', 0.0)
    print('case', p, r, K, N, dtype, flush=True)
    block, Z, H = 32, 2, 3
    layout = random_layout(H, p, r, 7 + p)
    layout[1] = layout[1, :1].expand(p, r)               # one head whose rows all share their columns
    if p > 4:
        layout[0, 4:8] = 0                               # an empty group
        layout[2, 1] = 0                                 # an empty row inside a group
    g = torch.Generator().manual_seed(5)
    a = torch.randn(Z, H, p * block, K, generator=g).to(dtype)
    b = torch.randn(Z, H, r * block, K, generator=g).to(dtype)
    c = matmul(layout, block, 'sdd', trans_b=True)(a.to(DEV), b.to(DEV))
    assert rel_err(c, ob.sdd(a, b, layout, block, trans_b=True)) <= TOL[dtype]
    nnz = int(layout.sum())
    sp = torch.randn(Z, nnz, block, block, generator=g).to(dtype)
    v = torch.randn(Z, H, r * block, N, generator=g).to(dtype)
    out = matmul(layout, block, 'dsd')(sp.to(DEV), v.to(DEV))
    assert rel_err(out, ob.dsd(sp, v, layout, block)) <= TOL[dtype]
    if p > 4:
        assert float(out[:, 0, 4 * block:8 * block].abs().max()) == 0.0
        assert float(out[:, 2, block:2 * block].abs().max()) == 0.0
    # the kernels without tile sharing give the same bits in SDD (same products, same order)
    monkeypatch.setattr(bm, 'UNION_MIN_SHARING', 1e9)
    c2 = matmul(layout, block, 'sdd', trans_b=True)(a.to(DEV), b.to(DEV))
    assert torch.equal(c, c2)


def test_config2_layout_stage_parity_reduced():
    """BASELINE config 2 pattern (band +-4 OR flat butterfly (8,2), block 32, bf16) at B=1, H=2."""
    from fly_amd import matmul, softmax, FlatBlockButterflySparsityConfig
    L, d, block = 4096, 64, 32
    lay = (FlatBlockButterflySparsityConfig(8, 2, block).make_layout(L) + ob.band_layout(L // block, L // block, 4)) > 0
    assert int(lay.sum()) == 6204
    layout = lay.long().unsqueeze(0).repeat(2, 1, 1)
    g = torch.Generator().manual_seed(0)
    q, k, v = (torch.randn(1, 2, L, d, generator=g).bfloat16() for _ in range(3))
    qk = matmul(layout, block, 'sdd', trans_b=True)(q.to(DEV), k.to(DEV))
    assert rel_err(qk, ob.sdd(q, k, layout, block, trans_b=True)) <= 2e-2
    p = softmax(layout, block)(qk.clone(), scale=0.125)
    assert rel_err(p, ob.block_softmax(qk.cpu(), layout, block, scale=0.125)) <= 2e-2
    out = matmul(layout, block, 'dsd')(p, v.to(DEV))
    assert rel_err(out, ob.dsd(p.cpu(), v, layout, block)) <= 2e-2


@pytest.mark.parametrize('Z', [8, 30])
def test_config2_full_size_heads_against_oracle(Z):
    """BASELINE config 2 at its full size (Z=8, H=12) and with a sparse tensor of more than 2^31
    elements (Z=30: 30 * 74448 * 1024 = 2.29e9): every stage of a few (batch, head) pairs, the last one
    of the tensor among them, against the oracle run on that pair alone; the one-kernel attention
    against the three stages over the whole output."""
    from fly_amd import matmul, softmax, FlatBlockButterflySparsityConfig
    from fly_amd.blocksparse_fused import fused_attention
    print('case', Z, flush=True)
    L, d, block, H = 4096, 64, 32, 12
    lay = ((FlatBlockButterflySparsityConfig(8, 2, block).make_layout(L) + ob.band_layout(L // block, L // block, 4)) > 0).long()
    per_head = int(lay.sum())
    assert per_head == 6204
    layout = lay.unsqueeze(0).repeat(H, 1, 1)
    torch.manual_seed(Z)
    q, k, v = (torch.randn(Z, H, L, d, device=DEV).bfloat16() for _ in range(3))
    qk = matmul(layout, block, 'sdd', trans_b=True)(q, k)
    assert qk.shape == (Z, H * per_head, block, block)
    if Z == 30:
        assert qk.numel() > 2 ** 31
    p = softmax(layout, block)(qk.clone(), scale=0.125)
    out = matmul(layout, block, 'dsd')(p, v)
    one = lay.unsqueeze(0)
    for z, h in [(0, 0), (Z // 2, 5), (Z - 1, H - 1)]:
        sl = slice(h * per_head, (h + 1) * per_head)
        qh, kh, vh = (t[z:z + 1, h:h + 1].cpu() for t in (q, k, v))
        qk_h = qk[z:z + 1, sl].cpu()
        assert rel_err(qk_h, ob.sdd(qh, kh, one, block, trans_b=True)) <= 2e-2
        p_h = p[z:z + 1, sl].cpu()
        assert rel_err(p_h, ob.block_softmax(qk_h, one, block, scale=0.125)) <= 2e-2
        assert rel_err(out[z:z + 1, h:h + 1], ob.dsd(p_h, vh, one, block)) <= 2e-2
    # size-independent property: every row of the softmax sums to one
    rows = p.view(Z, H, per_head, block, block).sum(-1, dtype=torch.float32)               # (Z, H, nnz, block)
    idx = lay.nonzero()[:, 0].to(DEV)                                                   # block-row of every block
    sums = torch.zeros(Z, H, L // block, block, device=DEV).index_add_(2, idx, rows)
    assert float((sums - 1).abs().max()) <= 2e-2
    del rows, sums, qk
    fused = fused_attention(layout, block)(q, k, v, 0.125)
    assert fused.shape == out.shape
    diff = float((fused.float() - out.float()).abs().max() / out.float().abs().max())
    assert diff <= 2e-2


@pytest.mark.parametrize('dtype,block', [(torch.float32, 16), (torch.float32, 32), (torch.bfloat16, 32)])
def test_sbblocksparse_attention_module(dtype, block):
    """Scatterbrain on a block-sparse support (sbblocksparse_attention.py:109-213): output, and with
    need_weights the dense attention matrix, against the oracle."""
    from fly_amd import SBBlockSparseAttention, FlatBlockButterflySparsityConfig
    from oracle import sbblocksparse as osbb
    print('case', dtype, block, flush=True)
    B, T, H, E = 2, 8 * block, 1, 64
    torch.manual_seed(0)
    layer = SBBlockSparseAttention(FlatBlockButterflySparsityConfig(4, 2, block=block), dim_heads=E,
                                   nb_features=64, max_seq_length=T).to(DEV)
    g = torch.Generator().manual_seed(4)
    q, k, v = (torch.randn(B, T, H, E, generator=g).to(dtype) for _ in range(3))
    q, k = q * E ** -0.25 * 2, k * E ** -0.25 * 2
    out, attn = layer(q.to(DEV), k.to(DEV), v.to(DEV), need_weights=True)
    P = layer.feature_map.projection_matrix.cpu().double()
    layout = layer.get_layout(T)
    ref_out, ref_ln = osbb.sbblocksparse_attention(q.double(), k.double(), v.double(), P, layout, block)
    tol = 1e-4 if dtype == torch.float32 else 2e-2
    assert out.shape == (B, T, H, E) and out.dtype == dtype
    assert rel_err(out, ref_out) <= tol
    # the attention matrix of the closed form: A / rowsum(A)
    _, _ = osbb.dense_closed_form(q.double(), k.double(), v.double(), P, layout, block)
    rows = attn.sum(-1)
    assert float((rows.float().cpu() - 1).abs().max()) <= (1e-4 if dtype == torch.float32 else 3e-2)
    ref_from_attn = torch.einsum('bhts,bshd->bthd', attn.double().cpu(), v.double())
    assert rel_err(ref_from_attn, ref_out) <= tol
    # without the weights: the fused kernels (the band kernel of Scatterbrain-local attention walking the layout's
    # blocks, 16 x 16 or 32 x 32)
    out2, none = layer(q.to(DEV), k.to(DEV), v.to(DEV))
    assert none is None and len(layer.fused_tables) == 1
    assert rel_err(out2, ref_out) <= tol
    layer.fuse = False
    out3, _ = layer(q.to(DEV), k.to(DEV), v.to(DEV))
    assert torch.equal(out3, out)


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16])
@pytest.mark.parametrize('p,r,D,rpg', [(8, 8, 64, 4), (13, 9, 64, 8), (5, 7, 32, 8), (6, 6, 128, 4), (9, 12, 128, 8)])
def test_fused_attention_matches_oracle(p, r, D, rpg, dtype):
    """One-kernel attention against the oracle's SDD -> softmax -> nan_to_num -> DSD in fp64 and
    against the three separate ops on the GPU; with an empty block-row, a key mask and queries
    whose keys are all masked."""
    from fly_amd import matmul, softmax
    from fly_amd.blocksparse_fused import fused_attention
    print('case', p, r, D, rpg, dtype, flush=True)
    Z, H, block = 2, 3, 32
    g = torch.Generator().manual_seed(100 * p + r)
    layout = random_layout(H, p, r, p * r, density=0.4)
    layout[1, min(2, p - 1), :] = 0                       # an empty block-row
    layout[0, 0, :] = 0
    layout[0, 0, 1] = 1                                   # a row whose only block is fully masked below
    q = torch.randn(Z, p * 32, H, D, generator=g).to(dtype)
    k = torch.randn(Z, r * 32, H, D, generator=g).to(dtype)
    v = torch.randn(Z, r * 32, H, D, generator=g).to(dtype)
    lens = torch.tensor([r * 32, 32])                     # batch 1 keeps only block-column 0
    kpm = torch.log((torch.arange(r * 32).view(1, -1) < lens.view(Z, 1)).float())
    scale = 0.31
    qh, kh, vh = (x.permute(0, 2, 1, 3) for x in (q, k, v))
    for mask in (None, kpm):
        qk = ob.sdd(qh.double(), kh.double(), layout, block, trans_b=True)
        pr = ob.block_softmax(qk, layout, block, scale=scale, key_padding_mask=mask).nan_to_num()
        ref = ob.dsd(pr, vh.double(), layout, block)
        op = fused_attention(layout, block, rows_per_group=rpg)
        out = op(qh.to(DEV), kh.to(DEV), vh.to(DEV), scale, None if mask is None else mask.to(DEV))
        assert out.shape == (Z, H, p * 32, D) and out.permute(0, 2, 1, 3).is_contiguous()
        assert rel_err(out, ref) <= TOL[dtype]
        assert float(out[:, 1, 32 * min(2, p - 1):32 * min(2, p - 1) + 32].abs().max()) == 0.0
        if mask is not None:
            assert float(out[1, 0, :32].abs().max()) == 0.0      # every key of that row is masked
        # the three separate kernels give the same result up to their extra roundings
        s3 = matmul(layout, block, 'sdd', trans_b=True)(qh.to(DEV), kh.to(DEV))
        a3 = softmax(layout, block)(s3, scale=scale, key_padding_mask=None if mask is None else mask.to(DEV))
        o3 = matmul(layout, block, 'dsd')(a3.nan_to_num_(), vh.to(DEV))
        assert rel_err(out, o3.float()) <= 2 * TOL[dtype]


def test_fused_attention_random_shapes():
    """Seeded random layouts, sizes, head dims, group sizes, dtypes, scales, key and attention masks against the
    oracle's SDD -> softmax -> nan_to_num -> DSD in float64: union lists of any length modulo the four block-columns a
    step takes, rows without blocks, heads without blocks, fully masked rows."""
    import random
    from fly_amd.blocksparse_fused import fused_attention
    rng = random.Random(20)
    for case in range(40):
        Z, H = rng.randint(1, 3), rng.randint(1, 3)
        p, r = rng.randint(1, 20), rng.randint(1, 20)
        D, rpg = rng.choice([32, 64, 128]), rng.choice([4, 8])
        dtype = rng.choice([torch.bfloat16, torch.float16])
        dens = rng.choice([0.1, 0.4, 0.8, 1.0])
        g = torch.Generator().manual_seed(case)
        layout = (torch.rand(H, p, r, generator=g) < dens).long()
        layout[0, 0, 0] = 1
        q = torch.randn(Z, p * 32, H, D, generator=g).to(dtype)
        k = torch.randn(Z, r * 32, H, D, generator=g).to(dtype)
        v = torch.randn(Z, r * 32, H, D, generator=g).to(dtype)
        kpm = am = None
        if rng.random() < 0.5:
            lens = torch.tensor([rng.randint(1, r * 32) for _ in range(Z)])
            kpm = torch.log((torch.arange(r * 32).view(1, -1) < lens.view(Z, 1)).float())
        if rng.random() < 0.3:
            am = torch.log((torch.rand(p * 32, r * 32, generator=g) < 0.7).float())
        scale = rng.choice([0.125, 0.31, 1.0])
        print('case', case, Z, H, p, r, D, rpg, dtype, dens, kpm is not None, am is not None, scale, flush=True)
        qh, kh, vh = (x.permute(0, 2, 1, 3) for x in (q, k, v))
        qk = ob.sdd(qh.double(), kh.double(), layout, 32, trans_b=True)
        pr = ob.block_softmax(qk, layout, 32, scale=scale, key_padding_mask=kpm, attn_mask=am).nan_to_num()
        ref = ob.dsd(pr, vh.double(), layout, 32)
        out = fused_attention(layout, 32, rows_per_group=rpg)(
            qh.to(DEV), kh.to(DEV), vh.to(DEV), scale, None if kpm is None else kpm.to(DEV),
            attn_mask=None if am is None else am.to(DEV))
        assert rel_err(out, ref) <= TOL[dtype], (case, rel_err(out, ref))


def test_fused_attention_with_an_empty_layout():
    """No nonzero block at all: zeros (the value of a row without blocks), and +inf as the rows' log-denominator."""
    from fly_amd.blocksparse_fused import fused_attention
    q, k, v = (torch.randn(2, 1, 64, 32, device=DEV).bfloat16() for _ in range(3))
    out, lse2 = fused_attention(torch.zeros(1, 2, 2, dtype=torch.long), 32)(q, k, v, 0.5, return_lse=True)
    assert out.shape == (2, 1, 64, 32) and float(out.abs().max()) == 0.0
    assert bool(torch.isinf(lse2).all())


def test_blocksparse_attention_module_fused_path():
    """BlockSparseAttention.forward takes the one-kernel path for eligible calls (eval / no grad, no
    attention mask) and the three-op path otherwise; both agree with the oracle, including padded
    sequence lengths and head dims (:107-127)."""
    from fly_amd import BlockSparseAttention, LengthMask

    class Cfg:
        block = 32

        def make_layout(self, seqlen):
            nb = seqlen // self.block
            lay = ob.band_layout(nb, nb, 1)
            lay[:, 0] = 1
            return lay.unsqueeze(0).repeat(2, 1, 1)

    B, T, S, H, E = 2, 300, 270, 2, 50
    g = torch.Generator().manual_seed(5)
    q = torch.randn(B, T, H, E, generator=g).bfloat16()
    k = torch.randn(B, S, H, E, generator=g).bfloat16()
    v = torch.randn(B, S, H, E, generator=g).bfloat16()
    lengths = torch.tensor([S, 101])
    mod = BlockSparseAttention(Cfg(), attention_dropout=0.0, max_seq_length=512).to(DEV)
    ref = ob.blocksparse_attention(q.double(), k.double(), v.double(), mod.master_layout.cpu(), 32, key_lengths=lengths)
    with torch.no_grad():
        out, w = mod(q.to(DEV), k.to(DEV), v.to(DEV), key_padding_mask=LengthMask(lengths.to(DEV), max_len=S))
    assert w is None and out.shape == (B, T, H, E)
    assert len(mod.fused_cache) == 1 and len(mod.ops_cache) == 0        # the fused kernel ran
    assert rel_err(out, ref) <= 2e-2
    mod.fuse = False
    out3, _ = mod(q.to(DEV), k.to(DEV), v.to(DEV), key_padding_mask=LengthMask(lengths.to(DEV), max_len=S))
    assert len(mod.ops_cache) == 1
    assert rel_err(out3, ref) <= 2e-2
    assert rel_err(out, out3.float()) <= 2e-2
    # a call that needs gradients keeps the differentiable three-op path
    mod.fuse = True
    mod.ops_cache.clear()
    qg = q.to(DEV).requires_grad_()
    outg, _ = mod(qg, k.to(DEV), v.to(DEV))
    assert len(mod.ops_cache) == 1
    outg.float().sum().backward()
    assert qg.grad is not None and bool(torch.isfinite(qg.grad.float()).all())


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16])
@pytest.mark.parametrize('p,r,D,rpg', [(7, 6, 64, 8), (5, 9, 32, 4), (9, 4, 128, 8)])
def test_fused_attention_with_attention_mask(p, r, D, rpg, dtype):
    """One-kernel attention with an additive (rows, cols) attention mask -- a random 0 / -inf mask, alone and
    together with a key mask, and a finite bias -- against the oracle's SDD -> softmax(attn_mask, mode 'add')
    -> nan_to_num -> DSD (blocksparse_attention.py:146-158); queries whose every score is masked give zero rows."""
    from fly_amd.blocksparse_fused import fused_attention
    print('case', p, r, D, rpg, dtype, flush=True)
    Z, H, block = 2, 3, 32
    g = torch.Generator().manual_seed(7 * p + r)
    layout = random_layout(H, p, r, 3 * p + r, density=0.5)
    layout[1, min(2, p - 1), :] = 0                       # an empty block-row
    q = torch.randn(Z, p * 32, H, D, generator=g).to(dtype)
    k = torch.randn(Z, r * 32, H, D, generator=g).to(dtype)
    v = torch.randn(Z, r * 32, H, D, generator=g).to(dtype)
    keep = torch.rand(p * 32, r * 32, generator=g) < 0.7
    keep[5] = False                                       # a query that may attend to nothing
    am_inf = torch.log(keep.float())
    am_bias = torch.randn(p * 32, r * 32, generator=g)
    lens = torch.tensor([r * 32, 40])
    kpm = torch.log((torch.arange(r * 32).view(1, -1) < lens.view(Z, 1)).float())
    scale = 0.27
    qh, kh, vh = (x.permute(0, 2, 1, 3) for x in (q, k, v))
    op = fused_attention(layout, block, rows_per_group=rpg)
    for am, km in ((am_inf, None), (am_inf, kpm), (am_bias, None)):
        qk = ob.sdd(qh.double(), kh.double(), layout, block, trans_b=True)
        pr = ob.block_softmax(qk, layout, block, scale=scale, key_padding_mask=km, attn_mask=am).nan_to_num()
        ref = ob.dsd(pr, vh.double(), layout, block)
        out = op(qh.to(DEV), kh.to(DEV), vh.to(DEV), scale, None if km is None else km.to(DEV), attn_mask=am.to(DEV))
        assert rel_err(out, ref) <= TOL[dtype]
        if am is am_inf:
            assert float(out[:, :, 5].abs().max()) == 0.0


def test_blocksparse_attention_module_fused_with_full_mask():
    """BlockSparseAttention.forward with a FullMask attention mask and a LengthMask stays on the one-kernel path
    (eval, no gradients, bf16, 32x32 blocks), with sequence lengths and head dims that need padding
    (blocksparse_attention.py:107-127,146-158; cf. tests/models/attention/test_blocksparse_attention.py:83-142)."""
    from fly_amd import BlockSparseAttention, FullMask, LengthMask

    class Cfg:
        block = 32

        def make_layout(self, seqlen):
            nb = seqlen // self.block
            lay = ob.band_layout(nb, nb, 1)
            lay[:, 0] = 1
            return lay.unsqueeze(0).repeat(3, 1, 1)

    B, T, S, H, E = 2, 235, 179, 3, 40
    g = torch.Generator().manual_seed(0)
    q = torch.randn(B, T, H, E, generator=g).bfloat16()
    k = torch.randn(B, S, H, E, generator=g).bfloat16()
    v = torch.randn(B, S, H, E, generator=g).bfloat16()
    lengths = torch.tensor([S, 77])
    am_bool = torch.rand(T, S, generator=g) < 0.8
    mod = BlockSparseAttention(Cfg(), attention_dropout=0.0, max_seq_length=256).to(DEV).eval()
    with torch.no_grad():
        out, w = mod(q.to(DEV), k.to(DEV), v.to(DEV), attn_mask=FullMask(am_bool.to(DEV)),
                     key_padding_mask=LengthMask(lengths.to(DEV), max_len=S))
    assert w is None and out.shape == (B, T, H, E)
    assert len(mod.fused_cache) == 1 and len(mod.ops_cache) == 0        # the fused kernel ran
    ref = ob.blocksparse_attention(q.double(), k.double(), v.double(), mod.master_layout.cpu(), 32,
                                   key_lengths=lengths, attn_mask_bool=am_bool)
    assert rel_err(out, ref) <= 2e-2
    mod.fuse = False
    with torch.no_grad():
        out3, _ = mod(q.to(DEV), k.to(DEV), v.to(DEV), attn_mask=FullMask(am_bool.to(DEV)),
                      key_padding_mask=LengthMask(lengths.to(DEV), max_len=S))
    assert rel_err(out, out3.float()) <= 2e-2


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16])
@pytest.mark.parametrize('p,r,K', [(8, 6, 1024), (5, 7, 2000), (12, 3, 777 * 16)])
def test_sdd_with_contraction_major_operands(p, r, K, dtype):
    """sparse = a^T b with a (K, M), b (K, N) and a long K -- the weight gradient of a block-sparse linear
    layer -- on the split-K kernel (fp32 accumulation over slices of K), with rows that share column
    lists (groups of up to four), rows that do not, an empty row, and K not a multiple of the step."""
    from fly_amd import matmul
    print('case', p, r, K, dtype, flush=True)
    Z, H, block = (2 if K < 2000 else 1), 2, 32
    layout = random_layout(H, p, r, 17 * p + r, density=0.5)
    layout[0, :4] = layout[0, 0]                          # a group of four rows with one column list
    layout[1, min(2, p - 1)] = 0                          # an empty block-row
    g = torch.Generator().manual_seed(K)
    a = torch.randn(Z, H, K, p * block, generator=g).to(dtype)
    b = torch.randn(Z, H, K, r * block, generator=g).to(dtype)
    op = matmul(layout, block, 'sdd', trans_a=True, trans_b=False)
    out = op(a.to(DEV), b.to(DEV))
    ref = ob.sdd(a.double(), b.double(), layout, block, trans_a=True, trans_b=False)
    assert out.shape == ref.shape and out.dtype == dtype
    assert rel_err(out, ref) <= TOL[dtype]
    # a layout without any block: an empty result, whichever kernel the shape would have selected
    empty = matmul(torch.zeros_like(layout), block, 'sdd', trans_a=True, trans_b=False)(a.to(DEV), b.to(DEV))
    assert empty.shape == (Z, 0, block, block)


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16])
@pytest.mark.parametrize('trans_b', [True, False])
def test_fast_dds_both_block_orientations(trans_b, dtype):
    """dense = x . op(sparse) on the tiled kernel for 2-byte types: blocks read as they are (y = x W^T,
    the forward of the Pixelfly linear) and transposed on their way into LDS (dx = dy W, its input
    gradient); token counts that are not multiples of the tile, grouped and ungrouped segments."""
    from fly_amd import matmul
    print('case', trans_b, dtype, flush=True)
    Z, H, block, p, r, M = 1, 2, 32, 9, 7, 333
    layout = random_layout(H, p, r, 23, density=0.5)
    layout[0, :3] = layout[0, 0]
    layout[1, :, 1] = 0                                   # an empty block-column
    g = torch.Generator().manual_seed(9)
    nnz = int(layout.sum())
    w = torch.randn(Z, nnz, block, block, generator=g).to(dtype)
    x = torch.randn(Z, H, M, (r if trans_b else p) * block, generator=g).to(dtype)
    out = matmul(layout, block, 'dds', trans_a=False, trans_b=trans_b)(x.to(DEV), w.to(DEV))
    ref = ob.dds(x.double(), w.double(), layout, block, False, trans_b)
    assert out.shape == ref.shape
    assert rel_err(out, ref) <= TOL[dtype]


@pytest.mark.parametrize('trans_b', [True, False])
def test_fast_dds_many_token_tiles_per_workgroup(trans_b):
    """The tiled dds kernel walks several 128-token tiles per workgroup once there are more tiles than
    workgroups wanted: enough tokens for two to three tiles each, a ragged last tile, an empty
    block-row (no input block at all) among the outputs."""
    from fly_amd import matmul
    print('case', trans_b, flush=True)
    Z, H, block, p, r, M = 1, 1, 32, 4, 3, 128 * 2500 + 37
    layout = torch.tensor([[[1, 0, 1], [1, 0, 1], [0, 1, 1], [1, 1, 0]]])
    if trans_b:
        layout[0, 1] = 0
    else:
        layout[0, :, 1] = 0
    g = torch.Generator().manual_seed(10)
    nnz = int(layout.sum())
    w = torch.randn(Z, nnz, block, block, generator=g).bfloat16()
    x = torch.randn(Z, H, M, (r if trans_b else p) * block, generator=g).bfloat16()
    out = matmul(layout, block, 'dds', trans_a=False, trans_b=trans_b)(x.to(DEV), w.to(DEV))
    ref = ob.dds(x.float(), w.float(), layout, block, False, trans_b)
    assert out.shape == ref.shape
    assert rel_err(out, ref) <= TOL[torch.bfloat16]


@pytest.mark.parametrize('trans_b', [True, False])
def test_tiled_dds_with_long_odd_reduction_lists(trans_b):
    """The tiled dds kernel takes two entries of a reduction list per step: lists of 10 to 12 input blocks (too long for
    the weight-stationary kernel; odd lengths end on a step with one entry), neighbouring and scattered input blocks,
    groups of one to four output blocks, a few thousand tokens (several tiles per workgroup) ending inside a tile."""
    from fly_amd import matmul
    print('case', trans_b, flush=True)
    Z, H, block, n_out, n_in, M = 2, 2, 32, 7, 13, 128 * 21 + 5
    g = torch.Generator().manual_seed(41)
    seg = (torch.rand(H, n_out, n_in, generator=g) < 0.85).long()   # (head, output block, input block)
    seg[0, 0] = 1
    seg[0, 0, 4] = 0                                       # 12 entries
    seg[0, 1:3] = seg[0, 0]                                # a group of three
    seg[1, 3, ::2] = 1
    seg[1, 3, 1::2] = (torch.arange(6) < 4).long()         # 11 entries, half of them without a neighbour
    assert int(seg.sum(-1).max()) > 9 and int(seg.sum(-1).min()) > 9 and bool((seg.sum(-1) % 2 == 1).any())
    layout = seg if trans_b else seg.transpose(1, 2).contiguous()
    w = torch.randn(Z, int(layout.sum()), block, block, generator=g).bfloat16()
    x = torch.randn(Z, H, M, n_in * block, generator=g).bfloat16()
    out = matmul(layout, block, 'dds', trans_a=False, trans_b=trans_b)(x.to(DEV), w.to(DEV))
    ref = ob.dds(x.float(), w.float(), layout, block, False, trans_b)
    assert out.shape == ref.shape == (Z, H, M, n_out * block)
    assert rel_err(out, ref) <= TOL[torch.bfloat16]


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16])
@pytest.mark.parametrize('trans_b', [True, False])
@pytest.mark.parametrize('M', [2048 + 77, 4096 + 1024 + 77])
def test_dds_weight_stationary_kernel(M, trans_b, dtype):
    """Reduction lists of at most nine blocks and a few thousand tokens: the dds kernels that keep a group's weights in
    LDS -- with activation fragments straight from memory (from 2048 tokens) and with the activations staged through
    LDS by direct-to-LDS transfers of whole 128-byte pieces of token rows (from 4096 tokens).  Two batch entries, two
    heads, groups of one to four segments (the last lanes of a short group store nothing), lists of odd and even
    length with neighbouring and scattered input blocks, a segment without blocks, a token count that ends inside a
    tile, both block orientations."""
    from fly_amd import matmul
    print('case', M, trans_b, dtype, flush=True)
    Z, H, block = 2, 2, 32
    p, r = (11, 9) if trans_b else (9, 11)                # segments: the output blocks, 11 of them either way
    g = torch.Generator().manual_seed(31)
    seg = (torch.rand(H, 11, 9, generator=g) < 0.45).long()   # (head, output block, input block): lists of <= 9
    seg[0, 1:4] = seg[0, 0]                                # a full group of four
    seg[1, 5:7] = seg[1, 4]                                # a group of three
    seg[1, 9] = 0                                          # an output block without inputs
    layout = seg if trans_b else seg.transpose(1, 2).contiguous()
    nnz = int(layout.sum())
    w = torch.randn(Z, nnz, block, block, generator=g).to(dtype)
    x = torch.randn(Z, H, M, 9 * block, generator=g).to(dtype)
    out = matmul(layout, block, 'dds', trans_a=False, trans_b=trans_b)(x.to(DEV), w.to(DEV))
    ref = ob.dds(x.double(), w.double(), layout, block, False, trans_b)
    assert out.shape == ref.shape == (Z, H, M, 11 * block)
    assert rel_err(out, ref) <= TOL[dtype]
    assert float(out[1, 1, :, 9 * block:10 * block].abs().max()) == 0.0


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16])
@pytest.mark.parametrize('trans_b', [True, False])
def test_dds_staged_kernel_with_weights_in_chunks(trans_b, dtype):
    """Reduction lists longer than nine blocks and more than 4096 tokens: the staged dds kernel whose group weights
    pass through LDS in double-buffered chunks of four list entries.  Lists of 10 to 21 entries (the last chunk of a
    list holds one to four entries, odd lengths end on a step with one entry), groups of one to four output blocks
    (the lanes of a short group store fewer outputs), two batch entries, two heads, a token count that ends inside a
    tile, both block orientations."""
    from fly_amd import matmul
    print('case', trans_b, dtype, flush=True)
    Z, H, block, n_out, n_in, M = 2, 2, 32, 10, 21, 4096 + 1024 + 77
    g = torch.Generator().manual_seed(43)
    seg = (torch.rand(H, n_out, n_in, generator=g) < 0.7).long()    # (head, output block, input block)
    seg[0, 0] = 1                                          # 21 entries: five chunks and one entry more
    seg[0, 1:4] = seg[0, 0]                                # a full group of four
    seg[0, 4] = (torch.arange(n_in) % 2 == 0).long()       # 11 entries, none with a neighbour
    seg[1, 0, :] = 0
    seg[1, 0, :10] = 1                                     # 10 entries: two chunks and half a chunk
    seg[1, 1:3] = seg[1, 0]                                # a group of three
    seg[1, 3] = (torch.arange(n_in) < 17).long()           # 17 entries: the last chunk holds one
    lens = seg.sum(-1)
    assert int(lens.max()) == 21 and all(bool((lens % 4 == k).any()) for k in range(4))
    layout = seg if trans_b else seg.transpose(1, 2).contiguous()
    w = torch.randn(Z, int(layout.sum()), block, block, generator=g).to(dtype)
    x = torch.randn(Z, H, M, n_in * block, generator=g).to(dtype)
    out = matmul(layout, block, 'dds', trans_a=False, trans_b=trans_b)(x.to(DEV), w.to(DEV))
    ref = ob.dds(x.double(), w.double(), layout, block, False, trans_b)
    assert out.shape == ref.shape == (Z, H, M, n_out * block)
    assert rel_err(out, ref) <= TOL[dtype]


@pytest.mark.parametrize('dtype', [torch.bfloat16, torch.float16])
@pytest.mark.parametrize('p,r,N', [(8, 8, 64), (11, 6, 72), (5, 13, 128)])
def test_dsd_with_transposed_sparse_operand(p, r, N, dtype):
    """dense = sparse^T . dense (dV = P^T dO, and dK = dS^T Q which arrives as a transposed dds) on the
    tiled kernel: groups of four block-columns share the dense tiles, every block is turned through
    LDS.  Band-like layouts (neighbouring columns share rows) so that the shared-tile path is taken."""
    from fly_amd import matmul
    print('case', p, r, N, dtype, flush=True)
    Z, H, block = 2, 2, 32
    rows = torch.arange(p).view(-1, 1) * r // p
    layout = ((rows - torch.arange(r).view(1, -1)).abs() <= 2).long().unsqueeze(0).repeat(H, 1, 1)
    layout[1, :, r - 1] = 0                               # an empty block-column
    nnz = int(layout.sum())
    g = torch.Generator().manual_seed(p * r)
    sp = torch.randn(Z, nnz, block, block, generator=g).to(dtype)
    dn = torch.randn(Z, H, p * block, N, generator=g).to(dtype)
    op = matmul(layout, block, 'dsd', trans_a=True, trans_b=False)
    out = op(sp.to(DEV), dn.to(DEV))
    ref = ob.dsd(sp.double(), dn.double(), layout, block, trans_a=True, trans_b=False)
    assert out.shape == ref.shape == (Z, H, r * block, N)
    assert rel_err(out, ref) <= TOL[dtype]
    assert float(out[:, 1, (r - 1) * block:].abs().max()) == 0.0
    # the same numbers through the dds form the backward pass of an sdd produces: (a^T b)^T
    a = dn.transpose(2, 3).contiguous()                   # (Z, H, N, p*block): op(a) = a is (N x K)
    out2 = matmul(layout, block, 'dds', trans_a=False, trans_b=False)(a.to(DEV), sp.to(DEV))
    ref2 = ob.dds(a.double(), sp.double(), layout, block, False, False)
    assert rel_err(out2, ref2) <= TOL[dtype]
    assert rel_err(out2.transpose(2, 3), ref) <= TOL[dtype]


@pytest.mark.parametrize('masked,E,dtype', [(True, 64, torch.bfloat16), (False, 64, torch.bfloat16), (False, 32, torch.bfloat16),
                                            (False, 128, torch.bfloat16), (False, 64, torch.float16), (True, 32, torch.float16),
                                            (True, 128, torch.bfloat16)])
def test_blocksparse_attention_module_gradients(masked, E, dtype):
    """Training path of BlockSparseAttention for 2-byte inputs: one autograd node; gradients against autograd through
    the oracle in float64 on the same rounded inputs.  The forward is the one-kernel attention and the backward forms
    the probabilities again from the rows' log-denominators -- per block, without writing them, for head dims up to 64
    (with padded keys the backward kernels read the key mask too); at 128 dims dV, the fused score gradient, dQ and dK on
    the tiled kernels."""
    from fly_amd import BlockSparseAttention, LengthMask

    class Cfg:
        block = 32

        def make_layout(self, seqlen):
            nb = seqlen // self.block
            lay = ob.band_layout(nb, nb, 2)
            lay[:, 0] = 1
            return lay.unsqueeze(0).repeat(2, 1, 1)

    B, T, H = 2, 384, 2
    print('case', masked, E, dtype, flush=True)
    g = torch.Generator().manual_seed(8)
    q, k, v = (torch.randn(B, T, H, E, generator=g).to(dtype) for _ in range(3))
    w = torch.randn(B, T, H, E, generator=g)
    lengths = torch.tensor([T, 200]) if masked else None
    mod = BlockSparseAttention(Cfg(), attention_dropout=0.0, max_seq_length=512).to(DEV)
    qd, kd, vd = (x.double().requires_grad_() for x in (q, k, v))
    ref = ob.blocksparse_attention(qd, kd, vd, mod.master_layout.cpu(), 32, key_lengths=lengths)
    (ref * w.double()).sum().backward()
    qg, kg, vg = (x.to(DEV).requires_grad_() for x in (q, k, v))
    out, _ = mod(qg, kg, vg, key_padding_mask=LengthMask(lengths.to(DEV), max_len=T) if masked else None)
    assert (len(mod.fused_cache) == 1) == (not masked or E <= 64)      # (with masks: the backward kernels that read them)
    seen, todo = set(), [out.grad_fn]
    while todo:                                           # the node sits behind the views that un-pad the output
        fn = todo.pop()
        if fn is None or fn in seen:
            continue
        seen.add(fn)
        todo += [f for f, _ in fn.next_functions]
    assert any('AttentionCore' in type(fn).__name__ for fn in seen)
    assert rel_err(out, ref) <= 2e-2
    (out.float() * w.to(DEV)).sum().backward()
    for got, want, name in ((qg.grad, qd.grad, 'dq'), (kg.grad, kd.grad, 'dk'), (vg.grad, vd.grad, 'dv')):
        assert rel_err(got.float(), want) <= 3e-2, (name, rel_err(got.float(), want))
    if masked:
        assert float(kg.grad[1, 200:].abs().max()) == 0.0


@pytest.mark.parametrize('E,dtype,nb', [(64, torch.bfloat16, 13), (32, torch.float16, 13), (64, torch.float16, 6),
                                          (32, torch.bfloat16, 22)])
def test_blocksparse_attention_gradients_without_stored_probabilities(E, dtype, nb, monkeypatch):
    """The backward after the one-kernel forward (flyhip_bs_attn_bwd: query-major launch for d query, key-major launch
    for d key and d value, probabilities and score gradients formed per block and never written): ragged layouts that
    differ by head -- a band on one, a band plus scattered blocks on the other -- with a block-row without blocks (zero
    output, zero d query), a block-column without blocks (zero d key and d value), a number of block-rows that is no
    multiple of four; against autograd through the oracle in float64 on the same rounded inputs."""
    from fly_amd import BlockSparseAttention, _lib
    print('case', E, dtype, nb, flush=True)
    called, call = [], _lib.call
    monkeypatch.setattr(_lib, 'call', lambda name, *args: (called.append(name), call(name, *args))[1])
    g = torch.Generator().manual_seed(100 + nb)
    lay = torch.stack([ob.band_layout(nb, nb, 1), ((torch.rand(nb, nb, generator=g) < 0.3) | (ob.band_layout(nb, nb, 2) > 0)).long()])
    lay[0, 2, :] = 0                                      # a block-row without blocks
    lay[1, :, 3] = 0                                      # a block-column without blocks
    lay[:, nb - 1, nb - 1] = 1

    class Cfg:
        block = 32

        def make_layout(self, seqlen):
            return lay.clone()

    B, T, H = 2, 32 * nb, 2
    q, k, v = (torch.randn(B, T, H, E, generator=g).to(dtype) for _ in range(3))
    w = torch.randn(B, T, H, E, generator=g).to(dtype)
    mod = BlockSparseAttention(Cfg(), attention_dropout=0.0, max_seq_length=T).to(DEV)
    qd, kd, vd = (x.double().requires_grad_() for x in (q, k, v))
    ref = ob.blocksparse_attention(qd, kd, vd, lay, 32)
    (ref * w.double()).sum().backward()
    qg, kg, vg = (x.to(DEV).requires_grad_() for x in (q, k, v))
    out, _ = mod(qg, kg, vg)
    assert len(mod.fused_cache) == 1
    tol = 3e-2 if dtype == torch.bfloat16 else 4e-3
    assert rel_err(out, ref) <= tol
    out.backward(w.to(DEV))
    assert 'flyhip_bs_attn_bwd' in called and not any('dsoftmax' in name for name in called), called
    for got, want, name in ((qg.grad, qd.grad, 'dq'), (kg.grad, kd.grad, 'dk'), (vg.grad, vd.grad, 'dv')):
        assert got.dtype == dtype and rel_err(got.float(), want) <= tol, (name, rel_err(got.float(), want))
    assert float(out.detach()[:, 64:96, 0].abs().max()) == 0.0 and float(qg.grad[:, 64:96, 0].abs().max()) == 0.0
    assert float(kg.grad[:, 96:128, 1].abs().max()) == 0.0 and float(vg.grad[:, 96:128, 1].abs().max()) == 0.0


@pytest.mark.parametrize('dtype,dropout', [(torch.float32, 0.0), (torch.bfloat16, 0.3)])
def test_blocksparse_attention_gradients_with_fully_masked_rows(dtype, dropout):
    """Band-only layout plus a length mask: the query rows past the band of the last valid key see no key
    at all.  The three-op path under autograd (fp32 inputs, or training with dropout) must give finite
    gradients, zero on padded keys -- and, without dropout, the oracle's."""
    from fly_amd import BlockSparseAttention, LengthMask

    class Cfg:
        block = 32

        def make_layout(self, seqlen):
            nb = seqlen // self.block
            return ob.band_layout(nb, nb, 1).unsqueeze(0).repeat(2, 1, 1)

    B, T, H, E = 2, 256, 2, 64
    print('case', dtype, dropout, flush=True)
    g = torch.Generator().manual_seed(18)
    q, k, v = (torch.randn(B, T, H, E, generator=g).to(dtype) for _ in range(3))
    w = torch.randn(B, T, H, E, generator=g)
    lengths = torch.tensor([T, 70])              # batch 1: block-rows 4.. see only masked keys
    mod = BlockSparseAttention(Cfg(), attention_dropout=dropout, max_seq_length=T).to(DEV).train()
    qg, kg, vg = (x.to(DEV).requires_grad_() for x in (q, k, v))
    torch.manual_seed(0)
    out, _ = mod(qg, kg, vg, key_padding_mask=LengthMask(lengths.to(DEV), max_len=T))
    assert len(mod.fused_cache) == 0
    assert float(out[1, 128:].detach().abs().max()) == 0.0
    (out.float() * w.to(DEV)).sum().backward()
    for grad in (qg.grad, kg.grad, vg.grad):
        assert bool(torch.isfinite(grad).all())
    assert float(kg.grad[1, 70:].abs().max()) == 0.0 and float(vg.grad[1, 70:].abs().max()) == 0.0
    assert float(qg.grad[1, 128:].abs().max()) == 0.0
    if dropout == 0.0:
        # dense masked softmax in float64 whose rows without any visible key are zero rows (autograd through
        # the oracle's NaN -> 0 replacement would itself yield NaN there)
        qd, kd, vd = (x.double().requires_grad_() for x in (q, k, v))
        lay = ob.densify_tensor(torch.ones(1, int(mod.master_layout.sum()), 32, 32), mod.master_layout.cpu())[0].bool()
        vis = lay.unsqueeze(0) & (torch.arange(T).view(1, 1, 1, T) < lengths.view(B, 1, 1, 1))      # (B, H, T, S)
        s = torch.einsum('bthe,bshe->bhts', qd, kd) / math.sqrt(E)
        live = vis.any(-1, keepdim=True)
        p = torch.softmax(torch.where(live, s.masked_fill(~vis, float('-inf')), torch.zeros_like(s)), -1) * live
        ref = torch.einsum('bhts,bshd->bthd', p, vd)
        (ref * w.double()).sum().backward()
        assert rel_err(out, ref) <= 1e-4
        assert rel_err(out, ob.blocksparse_attention(q.double(), k.double(), v.double(), mod.master_layout.cpu(), 32,
                                                     key_lengths=lengths)) <= 1e-4
        for got, want in ((qg.grad, qd.grad), (kg.grad, kd.grad), (vg.grad, vd.grad)):
            assert rel_err(got, want) <= 1e-4, rel_err(got, want)


@pytest.mark.parametrize('dtype,E,with_attn_mask', [(torch.bfloat16, 64, False), (torch.float16, 32, True), (torch.bfloat16, 64, True)])
def test_blocksparse_attention_masked_gradients_without_stored_probabilities(dtype, E, with_attn_mask, monkeypatch):
    """Training with masks on the one-kernel forward and the backward that forms the probabilities again per block
    (flyhip_bs_attn_masks, flyhip_bs_attn_bwd with key_mask / attn_mask): a band-only layout plus a length mask, so that
    the query rows past the band of the last valid key see no key at all (zero output, zero gradients, nothing
    non-finite), optionally a FullMask attention mask that hides scattered pairs; output and gradients against a dense
    masked softmax in float64 whose rows without a visible key are zero rows."""
    from fly_amd import BlockSparseAttention, LengthMask, FullMask, _lib
    print('case', dtype, E, with_attn_mask, flush=True)
    called, call = [], _lib.call
    monkeypatch.setattr(_lib, 'call', lambda name, *args: (called.append(name), call(name, *args))[1])

    class Cfg:
        block = 32

        def make_layout(self, seqlen):
            nb = seqlen // self.block
            return ob.band_layout(nb, nb, 1).unsqueeze(0).repeat(2, 1, 1)

    B, T, H = 2, 256, 2
    g = torch.Generator().manual_seed(19)
    q, k, v = (torch.randn(B, T, H, E, generator=g).to(dtype) for _ in range(3))
    w = torch.randn(B, T, H, E, generator=g).to(dtype)
    lengths = torch.tensor([T, 70])              # batch 1: block-rows 4.. see only masked keys
    keep = torch.rand(T, T, generator=g) < 0.8 if with_attn_mask else torch.ones(T, T, dtype=torch.bool)
    keep[torch.arange(T), torch.arange(T)] = True
    mod = BlockSparseAttention(Cfg(), attention_dropout=0.0, max_seq_length=T).to(DEV).train()
    qg, kg, vg = (x.to(DEV).requires_grad_() for x in (q, k, v))
    out, _ = mod(qg, kg, vg, key_padding_mask=LengthMask(lengths.to(DEV), max_len=T),
                 attn_mask=FullMask(keep.to(DEV)) if with_attn_mask else None)
    assert len(mod.fused_cache) == 1
    assert float(out[1, 128:].detach().abs().max()) == 0.0
    out.backward(w.to(DEV))
    assert 'flyhip_bs_attn_bwd' in called and 'flyhip_bs_attn_masks' in called, called
    for grad in (qg.grad, kg.grad, vg.grad):
        assert bool(torch.isfinite(grad).all())
    assert float(kg.grad[1, 70:].abs().max()) == 0.0 and float(vg.grad[1, 70:].abs().max()) == 0.0
    assert float(qg.grad[1, 128:].abs().max()) == 0.0
    qd, kd, vd = (x.double().requires_grad_() for x in (q, k, v))
    lay = ob.densify_tensor(torch.ones(1, int(mod.master_layout.sum()), 32, 32), mod.master_layout.cpu())[0].bool()
    vis = lay.unsqueeze(0) & keep.view(1, 1, T, T) & (torch.arange(T).view(1, 1, 1, T) < lengths.view(B, 1, 1, 1))
    sc = torch.einsum('bthe,bshe->bhts', qd, kd) / math.sqrt(E)
    live = vis.any(-1, keepdim=True)
    p = torch.softmax(torch.where(live, sc.masked_fill(~vis, float('-inf')), torch.zeros_like(sc)), -1) * live
    ref = torch.einsum('bhts,bshd->bthd', p, vd)
    (ref * w.double()).sum().backward()
    tol = 3e-2 if dtype == torch.bfloat16 else 4e-3
    assert rel_err(out, ref) <= tol
    for got, want, name in ((qg.grad, qd.grad, 'dq'), (kg.grad, kd.grad, 'dk'), (vg.grad, vd.grad, 'dv')):
        assert rel_err(got.float(), want) <= tol, (name, rel_err(got.float(), want))


@pytest.mark.parametrize('E,dtype,p_drop', [(64, torch.bfloat16, 0.25), (32, torch.float16, 0.1), (128, torch.bfloat16, 0.5)])
def test_blocksparse_attention_dropout_inside_the_kernels(E, dtype, p_drop):
    """Training-mode dropout of BlockSparseAttention (blocksparse_attention.py:160, constructor default 0.1) on the
    one-kernel forward and the recomputing backward: the mask is a hash of (seed, batch, head, query, key), restated
    on the host (oracle.sblocal.dropout_keep), so output and gradients are compared with float64 autograd through
    softmax -> mask / (1 - p) -> product on the kernels' own mask.  The reference draws its mask from torch's
    generator; independent keeps with probability 1 - p are what both share."""
    from fly_amd import BlockSparseAttention
    from oracle.sblocal import dropout_keep

    class Cfg:
        block = 32

        def make_layout(self, seqlen):
            nb = seqlen // self.block
            lay = ob.band_layout(nb, nb, 2)
            lay[:, 0] = 1
            lay[5, :] = 1
            return lay.unsqueeze(0).repeat(2, 1, 1)

    B, T, H = 2, 352, 2
    print('case', E, dtype, p_drop, flush=True)
    g = torch.Generator().manual_seed(21)
    q, k, v = (torch.randn(B, T, H, E, generator=g).to(dtype) for _ in range(3))
    w = torch.randn(B, T, H, E, generator=g)
    mod = BlockSparseAttention(Cfg(), attention_dropout=p_drop, max_seq_length=T).to(DEV).train()
    qg, kg, vg = (x.to(DEV).requires_grad_() for x in (q, k, v))
    torch.manual_seed(5)
    out, _ = mod(qg, kg, vg)
    seed = mod.last_dropout_seed
    assert seed is not None and len(mod.fused_cache) == 1 and len(mod.ops_cache) == 1
    (out.float() * w.to(DEV)).sum().backward()

    qd, kd, vd = (x.double().requires_grad_() for x in (q, k, v))
    lay = ob.densify_tensor(torch.ones(1, int(mod.master_layout.sum()), 32, 32), mod.master_layout.cpu())[0].bool()
    s = torch.einsum('bthe,bshe->bhts', qd, kd) / math.sqrt(E)
    prob = torch.softmax(s.masked_fill(~lay.unsqueeze(0), float('-inf')), -1)
    mult = dropout_keep(seed, p_drop, B, H, T, T)
    kept = float((mult > 0)[:, lay].double().mean())
    assert abs(kept - (1 - p_drop)) < 0.01, kept
    ref = torch.einsum('bhts,bshd->bthd', prob * mult, vd)
    (ref * w.double()).sum().backward()
    tol = 2e-2 if dtype == torch.bfloat16 else 4e-3
    assert rel_err(out, ref) <= tol, rel_err(out, ref)
    for got, want, name in ((qg.grad, qd.grad, 'dq'), (kg.grad, kd.grad, 'dk'), (vg.grad, vd.grad, 'dv')):
        assert rel_err(got.float(), want) <= 1.5 * tol, (name, rel_err(got.float(), want))
    # without gradients the same module call is the same kernel with the same mask for the same seed
    torch.manual_seed(5)
    with torch.no_grad():
        again, _ = mod(qg, kg, vg)
    assert mod.last_dropout_seed == seed and torch.equal(again, out.detach())
    # another seed, another mask; evaluation mode: none
    with torch.no_grad():
        other, _ = mod(qg, kg, vg)
        plain, _ = mod.eval()(qg, kg, vg)
    assert mod.last_dropout_seed is None
    assert rel_err(other, ref) > 0.1
    assert rel_err(plain, torch.einsum('bhts,bshd->bthd', prob, vd).detach()) <= tol


def test_probabilities_from_log_denominators():
    """flyhip_bs_attn_lse + flyhip_bs_sdd_prob: the one-kernel attention's per-row log-denominators
    turn an sdd into the softmax probabilities (what the training path's backward starts from); against
    the oracle's block softmax, with an empty block-row."""
    from fly_amd import _lib, matmul
    from fly_amd.blocksparse_fused import fused_attention
    Z, H, p, r, D, block = 2, 3, 9, 7, 64, 32
    g = torch.Generator().manual_seed(77)
    rows = torch.arange(p).view(-1, 1) * r // p
    layout = ((rows - torch.arange(r).view(1, -1)).abs() <= 2).long().unsqueeze(0).repeat(H, 1, 1)     # neighbouring rows share columns
    layout[1, 2, :] = 0
    q = torch.randn(Z, H, p * block, D, generator=g).bfloat16()
    k = torch.randn(Z, H, r * block, D, generator=g).bfloat16()
    v = torch.randn(Z, H, r * block, D, generator=g).bfloat16()
    out, lse2 = fused_attention(layout, block)(q.to(DEV), k.to(DEV), v.to(DEV), 0.2, return_lse=True)
    assert lse2.shape == (Z, H, p * block) and bool(torch.isinf(lse2[:, 1, 2 * block:3 * block]).all())
    sdd = matmul(layout, block, 'sdd', trans_b=True)
    uni_ptr, uni_inner, uni_blk = sdd._table('union', torch.device(DEV))
    nnz = int(layout.sum())
    qd, kd = q.to(DEV), k.to(DEV)
    probs = torch.empty(Z, nnz, block, block, dtype=torch.bfloat16, device=DEV)
    _lib.call('flyhip_bs_sdd_prob', qd.data_ptr(), kd.data_ptr(), lse2.data_ptr(), probs.data_ptr(),
              uni_ptr.data_ptr(), uni_inner.data_ptr(), uni_blk.data_ptr(), nnz, H, p, Z, D, block,
              qd.stride(0), qd.stride(1), qd.stride(2), kd.stride(0), kd.stride(1), kd.stride(2),
              0.2, _lib.dtype_code(qd), _lib.stream_ptr(torch.device(DEV)))
    ref = ob.block_softmax(ob.sdd(q.float(), k.float(), layout, block, trans_b=True), layout, block, scale=0.2)
    assert rel_err(probs, ref.nan_to_num()) <= 2e-2


@pytest.mark.parametrize('B,H,T,S,E,D,m,seed', [(2, 2, 256, 256, 64, 64, 64, 1), (1, 3, 224, 352, 32, 32, 32, 2),
                                                (2, 1, 96, 64, 128, 128, 256, 3), (1, 2, 416, 160, 40, 24, 26, 4),
                                                (11, 3, 160, 192, 32, 32, 32, 5)])
def test_sbblocksparse_fused_forward(B, H, T, S, E, D, m, seed):
    """Scatterbrain attention on a block-sparse support on the fused kernels (flyhip_sbblocksparse_fwd): random
    layouts per head with an empty block-row, an odd number of block-rows (a query tile with one block-row),
    T != S, head dims and feature counts that need padding; output and log-normaliser against the oracle."""
    from fly_amd.blocksparse_utils import tile_mask_table, union_table
    from fly_amd.sblocal_attention import sbblocksparse_forward
    from oracle import sbblocksparse as osbb
    from oracle import sblocal as osb
    print('case', B, H, T, S, E, D, m, flush=True)
    g = torch.Generator().manual_seed(seed)
    layout = (torch.rand(H, T // 32, S // 32, generator=g) < 0.4).long()
    layout[:, :, 0] = 1
    layout[0, 1, :] = 0
    q = torch.randn(B, T, H, E, generator=g) * E ** -0.25
    k = torch.randn(B, S, H, E, generator=g) * E ** -0.25
    v = torch.randn(B, S, H, D, generator=g)
    P = osb.gaussian_orthogonal_random_matrix(m // 2, E, generator=g)
    tables = tuple(x.to(DEV) for x in tile_mask_table(layout, 32))
    out, ln = sbblocksparse_forward(q.to(DEV), k.to(DEV), v.to(DEV), P.to(DEV), tables)
    ref_out, ref_ln = osbb.sbblocksparse_attention(q.double(), k.double(), v.double(), P.double(), layout, 32)
    assert out.shape == (B, T, H, D) and ln.shape == (B, H, T, 1)
    assert rel_err(out, ref_out) <= 1e-4, rel_err(out, ref_out)
    assert rel_err(ln.reshape(ref_ln.shape), ref_ln) <= 1e-4, rel_err(ln.reshape(ref_ln.shape), ref_ln)
    # the same with the tiles started longest list first: every tile is still computed once, by the same code
    from fly_amd.blocksparse_utils import union_order
    ordered = tables + (union_order(tables[0], H).to(DEV),)
    out2, ln2 = sbblocksparse_forward(q.to(DEV), k.to(DEV), v.to(DEV), P.to(DEV), ordered)
    assert torch.equal(out2, out) and torch.equal(ln2, ln)


@pytest.mark.parametrize('B,H,T,S,E,D,m,seed', [(2, 2, 208, 144, 64, 64, 64, 11), (1, 3, 784, 784, 64, 64, 16, 12),
                                                (2, 1, 48, 400, 32, 48, 32, 13)])
def test_sbblocksparse_fused_forward_on_16x16_blocks(B, H, T, S, E, D, m, seed):
    """The fused forward on a support of 16 x 16 blocks (the block size of the reference's second T2T layer,
    configs/model/t2tattn_cfg/sbbs-*.yaml): a wave of the band kernel is one block-row, a 32-key tile two
    block-columns, each present or not.  Sequence lengths that are no multiples of 32 or 64, block-rows without
    blocks, a column of global keys; output and log-normaliser against the oracle."""
    from fly_amd.blocksparse_utils import tile_mask_table
    from fly_amd.sblocal_attention import sbblocksparse_forward
    from oracle import sbblocksparse as osbb
    from oracle import sblocal as osb
    print('case', B, H, T, S, E, D, m, seed, flush=True)
    g = torch.Generator().manual_seed(seed)
    layout = (torch.rand(H, T // 16, S // 16, generator=g) < 0.3).long()
    layout[:, :, 0] = 1
    layout[0, 1, :] = 0                                        # a block-row without blocks
    if T // 16 > 5:
        layout[-1, 5, :] = 0
    q = torch.randn(B, T, H, E, generator=g) * E ** -0.25
    k = torch.randn(B, S, H, E, generator=g) * E ** -0.25
    v = torch.randn(B, S, H, D, generator=g)
    P = osb.gaussian_orthogonal_random_matrix(m // 2, E, generator=g)
    tables = tuple(x.to(DEV) for x in tile_mask_table(layout, 16))
    out, ln = sbblocksparse_forward(q.to(DEV), k.to(DEV), v.to(DEV), P.to(DEV), tables)
    ref_out, ref_ln = osbb.sbblocksparse_attention(q.double(), k.double(), v.double(), P.double(), layout, 16)
    assert out.shape == (B, T, H, D) and ln.shape == (B, H, T, 1)
    assert rel_err(out, ref_out) <= 1e-4, rel_err(out, ref_out)
    assert rel_err(ln.reshape(ref_ln.shape), ref_ln) <= 1e-4, rel_err(ln.reshape(ref_ln.shape), ref_ln)


def test_sbblocksparse_fused_forward_with_an_empty_layout():
    """A support without any block: what remains is the low-rank estimate alone (linear attention on the features)."""
    from fly_amd.blocksparse_utils import tile_mask_table, union_table
    from fly_amd.sblocal_attention import sbblocksparse_forward
    from oracle import sbblocksparse as osbb
    from oracle import sblocal as osb
    g = torch.Generator().manual_seed(7)
    B, H, T, S, E, D, m = 2, 1, 32, 96, 64, 64, 64
    layout = torch.zeros(H, T // 32, S // 32, dtype=torch.long)
    q = torch.randn(B, T, H, E, generator=g) * E ** -0.25
    k = torch.randn(B, S, H, E, generator=g) * E ** -0.25
    v = torch.randn(B, S, H, D, generator=g)
    P = osb.gaussian_orthogonal_random_matrix(m // 2, E, generator=g)
    tables = tuple(x.to(DEV) for x in tile_mask_table(layout, 32))
    out, ln = sbblocksparse_forward(q.to(DEV), k.to(DEV), v.to(DEV), P.to(DEV), tables)
    ref_out, ref_ln = osbb.sbblocksparse_attention(q.double(), k.double(), v.double(), P.double(), layout, 32)
    assert rel_err(out, ref_out) <= 1e-4, rel_err(out, ref_out)
    assert rel_err(ln.reshape(ref_ln.shape), ref_ln) <= 1e-4


@pytest.mark.parametrize('B,H,T,S,E,D,m,seed,block', [(2, 2, 256, 256, 64, 64, 64, 1, 32), (1, 3, 224, 352, 32, 32, 32, 2, 32),
                                                      (1, 2, 416, 160, 40, 24, 26, 4, 32), (3, 1, 160, 192, 64, 64, 128, 5, 32),
                                                      (2, 2, 208, 144, 64, 64, 64, 6, 16), (1, 3, 784, 784, 64, 64, 16, 7, 16),
                                                      (2, 1, 48, 400, 32, 48, 32, 8, 16)])
def test_sbblocksparse_gradients_on_the_kernels(B, H, T, S, E, D, m, seed, block):
    """Gradients of Scatterbrain attention on a block-sparse support from the backward kernels walking the layout's
    blocks (flyhip_sblocal_bwd_prep, flyhip_sbblocksparse_bwd_pieces) against autograd through the oracle in float64
    (sbblocksparse_attention.py:161-212): random layouts per head with an empty block-row, an odd number of
    block-rows and block-columns, T != S, head dims and feature counts that need padding; 32 x 32 and 16 x 16 blocks (the
    latter with lengths that are not multiples of 32: half tiles past the end)."""
    from fly_amd import sblocal_backward
    from fly_amd.blocksparse_utils import tile_mask_table, union_table
    from fly_amd.sblocal_attention import sbblocksparse_forward
    from oracle import sbblocksparse as osbb
    from oracle import sblocal as osb
    print('case', B, H, T, S, E, D, m, block, flush=True)
    g = torch.Generator().manual_seed(seed)
    layout = (torch.rand(H, T // block, S // block, generator=g) < (0.4 if block == 32 else 0.2)).long()
    layout[:, :, 0] = 1
    layout[0, 1, :] = 0
    q = torch.randn(B, T, H, E, generator=g) * E ** -0.25
    k = torch.randn(B, S, H, E, generator=g) * E ** -0.25
    v = torch.randn(B, S, H, D, generator=g)
    w = torch.randn(B, T, H, D, generator=g)
    P = osb.gaussian_orthogonal_random_matrix(m // 2, E, generator=g)
    qd, kd, vd = (x.double().requires_grad_() for x in (q, k, v))
    ref_out, _ = osbb.sbblocksparse_attention(qd, kd, vd, P.double(), layout, block)
    (ref_out * w.double()).sum().backward()
    fwd = tuple(x.to(DEV) for x in tile_mask_table(layout, block))
    bwd = tuple(x.to(DEV) for x in tile_mask_table(layout, block, transposed=True))
    qg, kg, vg = q.to(DEV), k.to(DEV), v.to(DEV)
    out, ln = sbblocksparse_forward(qg, kg, vg, P.to(DEV), fwd)
    dq, dk, dv = sblocal_backward(qg, kg, vg, P.to(DEV), 1, None, None, out, ln, w.to(DEV), support=(fwd, bwd))
    for got, ref in ((dq, qd.grad), (dk, kd.grad), (dv, vd.grad)):
        assert got.shape == ref.shape and rel_err(got, ref) <= 2e-4, rel_err(got, ref)


@pytest.mark.parametrize('block,p_drop', [(32, 0.25), (16, 0.1)])
def test_sbblocksparse_dropout_inside_the_kernels(block, p_drop):
    """Training-mode dropout of SBBlockSparseAttention (sbblocksparse_attention.py:196-200: of the exact weights only)
    inside the fused forward and the backward kernels (32 x 32 and 16 x 16 blocks): the mask is the hash of (seed, batch,
    head, query, key) restated in oracle.sblocal.dropout_keep, handed to the oracle as nn.Dropout's multiplier."""
    from fly_amd import SBBlockSparseAttention, FlatBlockButterflySparsityConfig
    from oracle import sbblocksparse as osbb
    from oracle.sblocal import dropout_keep
    B, T, H, E = 2, 256, 1, 64
    print('case', block, p_drop, flush=True)
    torch.manual_seed(0)
    layer = SBBlockSparseAttention(FlatBlockButterflySparsityConfig(4, 2, block=block), dim_heads=E, nb_features=64,
                                   attention_dropout=p_drop, max_seq_length=T).to(DEV).train()
    g = torch.Generator().manual_seed(6)
    q, k, v, w = (torch.randn(B, T, H, E, generator=g) for _ in range(4))
    q, k = q * E ** -0.25 * 2, k * E ** -0.25 * 2
    train = True
    qg, kg, vg = (x.to(DEV).requires_grad_(train) for x in (q, k, v))
    torch.manual_seed(9)
    out, _ = layer(qg, kg, vg)
    seed = layer.last_dropout_seed
    assert seed is not None and len(layer.fused_tables) == 1 and len(layer.ops_cache) == 0
    P = layer.feature_map.projection_matrix.cpu().double()
    qd, kd, vd = (x.double().requires_grad_() for x in (q, k, v))
    mult = dropout_keep(seed, p_drop, B, H, T, T)
    ref_out, _ = osbb.sbblocksparse_attention(qd, kd, vd, P, layer.get_layout(T), block, dropout_multiplier=mult)
    assert rel_err(out, ref_out) <= 1e-4, rel_err(out, ref_out)
    plain_ref, _ = osbb.sbblocksparse_attention(qd, kd, vd, P, layer.get_layout(T), block)
    assert rel_err(out, plain_ref) > 1e-2
    if train:
        assert len(layer.backward_tables) == 1
        (out * w.to(DEV)).sum().backward()
        (ref_out * w.double()).sum().backward()
        for got, ref in ((qg.grad, qd.grad), (kg.grad, kd.grad), (vg.grad, vd.grad)):
            assert rel_err(got, ref) <= 2e-4, rel_err(got, ref)
    with torch.no_grad():
        plain, _ = layer.eval()(qg, kg, vg)
    assert layer.last_dropout_seed is None and rel_err(plain, plain_ref) <= 1e-4


def test_sbblocksparse_module_trains_on_the_fused_kernels():
    """SBBlockSparseAttention with gradients: the forward stays on the fused kernels and the backward walks the
    layout's blocks; gradients of query, key and value against autograd through the oracle, and against the op-by-op
    path of the same module."""
    from fly_amd import SBBlockSparseAttention, FlatBlockButterflySparsityConfig
    from oracle import sbblocksparse as osbb
    B, T, H, E, block = 2, 256, 1, 64, 32
    torch.manual_seed(0)
    layer = SBBlockSparseAttention(FlatBlockButterflySparsityConfig(4, 2, block=block), dim_heads=E,
                                   nb_features=64, max_seq_length=T).to(DEV)
    g = torch.Generator().manual_seed(4)
    q, k, v, w = (torch.randn(B, T, H, E, generator=g) for _ in range(4))
    q, k = q * E ** -0.25 * 2, k * E ** -0.25 * 2
    qg, kg, vg = (x.to(DEV).requires_grad_() for x in (q, k, v))
    out, _ = layer(qg, kg, vg)
    assert len(layer.backward_tables) == 1                  # the kernel path
    (out * w.to(DEV)).sum().backward()
    P = layer.feature_map.projection_matrix.cpu().double()
    qd, kd, vd = (x.double().requires_grad_() for x in (q, k, v))
    ref_out, _ = osbb.sbblocksparse_attention(qd, kd, vd, P, layer.get_layout(T), block)
    (ref_out * w.double()).sum().backward()
    assert rel_err(out, ref_out) <= 1e-4
    for got, ref in ((qg.grad, qd.grad), (kg.grad, kd.grad), (vg.grad, vd.grad)):
        assert rel_err(got, ref) <= 2e-4, rel_err(got, ref)
    layer.fuse = False
    q2, k2, v2 = (x.to(DEV).requires_grad_() for x in (q, k, v))
    out2, _ = layer(q2, k2, v2)
    (out2 * w.to(DEV)).sum().backward()
    for got, ref in ((qg.grad, q2.grad), (kg.grad, k2.grad), (vg.grad, v2.grad)):
        assert rel_err(got, ref) <= 2e-4, rel_err(got, ref)


def test_sbblocksparse_gradients_with_long_lists_in_parts():
    """Backward kernels on a support with block-rows and block-columns of global tokens: the outer tiles with long
    lists (queries of the global rows, keys of the global columns) are walked in parts and finished by a second
    launch (sbblocksparse_attention.backward_tables); gradients against autograd through the oracle and against the
    walk of whole lists."""
    from fly_amd import sblocal_backward
    from fly_amd.blocksparse_utils import tile_mask_table, union_table
    from fly_amd.sbblocksparse_attention import backward_tables
    from fly_amd.sblocal_attention import sbblocksparse_forward
    from oracle import sbblocksparse as osbb
    from oracle import sblocal as osb
    B, H, L, E, m = 2, 2, 1280, 64, 64
    nb = L // 32
    g = torch.Generator().manual_seed(12)
    idx = torch.arange(nb)
    window = ((idx[:, None] - idx[None, :]).abs() <= 1).long()
    layout = torch.stack([window.clone(), window.clone()])
    layout[0, 0, :] = 1                       # head 0: a global block-row and a global block-column
    layout[0, :, 0] = 1
    layout[1, 21, :] = 1                      # head 1: a global block-row in the second half of its tile,
    layout[1, :, 38:40] = 1                   # and a key tile whose two block-columns are both global
    q = torch.randn(B, L, H, E, generator=g) * E ** -0.25
    k = torch.randn(B, L, H, E, generator=g) * E ** -0.25
    v = torch.randn(B, L, H, E, generator=g)
    w = torch.randn(B, L, H, E, generator=g)
    P = osb.gaussian_orthogonal_random_matrix(m // 2, E, generator=g)
    tq, tk = backward_tables(layout, DEV), backward_tables(layout, DEV, transposed=True)
    assert sorted(tq[4].tolist()) == [0, 20 + 10] and sorted(tk[4].tolist()) == [0, 20 + 19]
    assert tq[5] >= 2 and tk[5] >= 2
    qd, kd, vd = (x.double().requires_grad_() for x in (q, k, v))
    ref_out, _ = osbb.sbblocksparse_attention(qd, kd, vd, P.double(), layout, 32)
    (ref_out * w.double()).sum().backward()
    qg, kg, vg = q.to(DEV), k.to(DEV), v.to(DEV)
    out, ln = sbblocksparse_forward(qg, kg, vg, P.to(DEV), tuple(x.to(DEV) for x in tile_mask_table(layout, 32)))
    got = sblocal_backward(qg, kg, vg, P.to(DEV), 1, None, None, out, ln, w.to(DEV), support=(tq, tk))
    for x, ref in zip(got, (qd.grad, kd.grad, vd.grad)):
        assert rel_err(x, ref) <= 2e-4, rel_err(x, ref)
    whole = sblocal_backward(qg, kg, vg, P.to(DEV), 1, None, None, out, ln, w.to(DEV), support=(tq[:3], tk[:3]))
    for x, y in zip(got, whole):
        assert rel_err(x, y) <= 1e-5, rel_err(x, y)


@pytest.mark.parametrize('dtype,block', [(torch.bfloat16, 32), (torch.float16, 32), (torch.bfloat16, 16), (torch.float16, 16)])
def test_sbblocksparse_forward_reads_2byte_tensors_as_they_are(dtype, block):
    """bfloat16 / float16 q, k, v go to the kernels on operand images without float32 copies (the key pass and the band
    kernel widen what they load, the band kernel and the merge of long lists round what they store): the arithmetic is the
    float32 path's on the same values, so the output equals the float32 path's output rounded, bit for bit, and the
    log-normaliser is the same.  Supports with a block-row of global tokens (a long list walked in parts and merged) and
    windows, two heads that differ; against the oracle on the rounded inputs as well; through the module too."""
    from fly_amd import SBBlockSparseAttention
    from fly_amd.sbblocksparse_attention import fused_tables
    from fly_amd.sblocal_attention import sbblocksparse_forward
    from oracle import sbblocksparse as osbb
    from oracle import sblocal as osb
    print('case', dtype, block, flush=True)
    B, H, L, E, m = 2, 2, 40 * block, 64, 64
    nb = L // block
    g = torch.Generator().manual_seed(13)
    idx = torch.arange(nb)
    window = ((idx[:, None] - idx[None, :]).abs() <= 1).long()
    layout = torch.stack([window.clone(), window.clone()])
    layout[0, 0, :] = 1
    layout[0, :, 0] = 1
    layout[1, 21, :] = 1
    q, k, v = (torch.randn(B, L, H, E, generator=g) for _ in range(3))
    q, k = (q * E ** -0.25).to(dtype), (k * E ** -0.25).to(dtype)
    v = v.to(dtype)
    P = osb.gaussian_orthogonal_random_matrix(m // 2, E, generator=g)
    tables = fused_tables(layout, DEV, block)
    out, ln = sbblocksparse_forward(q.to(DEV), k.to(DEV), v.to(DEV), P.to(DEV), tables)
    assert out.dtype == dtype and ln.dtype == torch.float32
    wide, ln_w = sbblocksparse_forward(q.float().to(DEV), k.float().to(DEV), v.float().to(DEV), P.to(DEV), tables)
    assert torch.equal(out, wide.to(dtype)) and torch.equal(ln, ln_w)
    ref_out, ref_ln = osbb.sbblocksparse_attention(q.double(), k.double(), v.double(), P.double(), layout, block)
    assert rel_err(out, ref_out) <= (1e-2 if dtype == torch.bfloat16 else 2e-3)
    assert rel_err(ln.reshape(ref_ln.shape), ref_ln) <= 1e-4

    class Cfg:
        def __init__(self):
            self.block = block

        def make_layout(self, seqlen):
            return layout.clone()

    layer = SBBlockSparseAttention(Cfg(), dim_heads=E, nb_features=m, max_seq_length=L).to(DEV).eval()
    with torch.no_grad():
        layer(q.to(DEV), k.to(DEV), v.to(DEV))                     # (the first call draws the projection)
        layer.feature_map.projection_matrix.copy_(P)
        got, _ = layer(q.to(DEV), k.to(DEV), v.to(DEV))
    assert got.dtype == dtype and torch.equal(got, out)


def test_sbblocksparse_long_lists_in_parts():
    """Block-rows of global tokens: their query tiles' lists are walked in parts by a second launch and merged
    (fused_tables marks them); output and log-normaliser against the oracle and against the one-part path."""
    from fly_amd.blocksparse_utils import tile_mask_table, union_table
    from fly_amd.sbblocksparse_attention import fused_tables
    from fly_amd.sblocal_attention import sbblocksparse_forward
    from oracle import sbblocksparse as osbb
    from oracle import sblocal as osb
    B, H, L, E, m = 3, 2, 1280, 64, 64
    nb = L // 32
    g = torch.Generator().manual_seed(11)
    idx = torch.arange(nb)
    window = ((idx[:, None] - idx[None, :]).abs() <= 1).long()
    layout = torch.stack([window.clone(), window.clone()])
    layout[0, 0, :] = 1                       # head 0: block-row 0 global (tile 0: 40 entries, its second row a window)
    layout[0, :, 0] = 1
    layout[1, 21, :] = 1                      # head 1: block-row 21 global (second row of tile 10)
    layout[1, 38:40, :] = 1                   # and a tile whose two rows are both long
    q = torch.randn(B, L, H, E, generator=g) * E ** -0.25
    k = torch.randn(B, L, H, E, generator=g) * E ** -0.25
    v = torch.randn(B, L, H, E, generator=g)
    P = osb.gaussian_orthogonal_random_matrix(m // 2, E, generator=g)
    tables = fused_tables(layout, DEV)
    assert sorted(tables[4].tolist()) == [0, 20 + 10, 20 + 19] and tables[5] >= 2
    assert sorted(-1 - x for x in tables[3].tolist() if x < 0) == [0, 10, 19]
    print('case long lists', tables[4].tolist(), tables[5], flush=True)
    out, ln = sbblocksparse_forward(q.to(DEV), k.to(DEV), v.to(DEV), P.to(DEV), tables)
    ref_out, ref_ln = osbb.sbblocksparse_attention(q.double(), k.double(), v.double(), P.double(), layout, 32)
    assert rel_err(out, ref_out) <= 1e-4, rel_err(out, ref_out)
    assert rel_err(ln.reshape(ref_ln.shape), ref_ln) <= 1e-4, rel_err(ln.reshape(ref_ln.shape), ref_ln)
    plain = tuple(x.to(DEV) for x in tile_mask_table(layout, 32))
    out1, ln1 = sbblocksparse_forward(q.to(DEV), k.to(DEV), v.to(DEV), P.to(DEV), plain)
    assert rel_err(out, out1) <= 1e-5 and rel_err(ln, ln1) <= 1e-5
