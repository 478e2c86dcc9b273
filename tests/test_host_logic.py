"""CPU-side checks of the product package: host logic is bit-exact against the oracle, the
reference's error behaviour is mirrored, and the C-ABI library loads and exports every symbol the
header declares.  Nothing here launches a kernel."""
import ctypes
import os
import re

import pytest
import torch

import fly_amd
from fly_amd import _lib
from fly_amd import blocksparse_utils as bu
from oracle import blocksparse as ob

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _layout(H, p, r, seed, density=0.5):
    g = torch.Generator().manual_seed(seed)
    return (torch.rand(H, p, r, generator=g) < density).long()


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, 'include', 'flyhip.h')).read()
    declared = set(re.findall(r'\b(flyhip_\w+)\s*\(', header))
    assert {'flyhip_sb_kv_reduce', 'flyhip_sblocal_fwd', 'flyhip_local_fwd', 'flyhip_bs_sdd', 'flyhip_bs_dsd', 'flyhip_bs_dds',
            'flyhip_bs_softmax', 'flyhip_bs_softmax_bwd', 'flyhip_bs_attn', 'flyhip_bs_sdd_kmajor', 'flyhip_bs_sdd_dsoftmax', 'flyhip_bs_rowreduce', 'flyhip_sb_plan', 'flyhip_version',
            'flyhip_last_error'} <= declared
    lib = _lib.load()
    for name in declared:
        assert hasattr(lib, name), f'{name} declared in include/flyhip.h but not exported'
    assert set(_lib.SIGNATURES) | {'flyhip_last_error', 'flyhip_sb_workspace_bytes', 'flyhip_sblocal_bwd_prep_scratch', 'flyhip_sblocal_bwd_image_bytes', 'flyhip_sblocal_bwd_parts_floats', 'flyhip_sbblocksparse_bwd_parts_floats'} == declared
    assert lib.flyhip_version() >= 100
    # pure host entry point: the launch plan
    nc, ns, npart = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    _lib.call('flyhip_sb_plan', 2, 1, 3136, 3136, 512, ctypes.byref(nc), ctypes.byref(ns), ctypes.byref(npart))
    assert nc.value == 49 and 1 <= ns.value <= 49 and 1 <= npart.value <= 8
    with pytest.raises(RuntimeError, match='bad arguments'):
        _lib.call('flyhip_sb_plan', 0, 1, 10, 10, 4, ctypes.byref(nc), ctypes.byref(ns), ctypes.byref(npart))
    # the first T2T layer (B=64, L=3136): 49 chunks a head; the fp32 key pass on bf16 pieces holds one workgroup per
    # compute unit, so one full round of 256 workgroups (4 a head, 13 chunks each) beats two rounds of 7 chunks
    _lib.call('flyhip_sb_plan_for', 64, 1, 3136, 3136, 256, 64, 64, 0, ctypes.byref(nc), ctypes.byref(ns), ctypes.byref(npart))
    assert (nc.value, ns.value, npart.value) == (49, 4, 1)
    _lib.call('flyhip_sb_plan_for', 64, 1, 3136, 3136, 256, 64, 64, 1, ctypes.byref(nc), ctypes.byref(ns), ctypes.byref(npart))
    assert (nc.value, ns.value) == (49, 7)


@pytest.mark.parametrize('args', [(3072, 768, 8, 2, 32), (768, 3072, 8, 2, 32), (4096, 4096, 8, 2, 32),
                                  (1024, 512, 16, 2, 32), (512, 512, 8, 3, 16), (256, 256, 8, 2, 32)])
@pytest.mark.parametrize('extra', [{}, {'global_size': 32}, {'shuffle': True}])
def test_flat_butterfly_layout_bit_exact(args, extra):
    out_f, in_f, bs, nf, blk = args
    cfg = fly_amd.FlatBlockButterflySparsityConfig(bs, nf, block=blk, **extra)
    got = cfg.make_layout(out_f, in_f)
    want = ob.flat_butterfly_layout(out_f, in_f, bs, nf, blk, **extra)
    assert got.dtype == want.dtype == torch.int32 and torch.equal(got, want)
    with pytest.raises(NotImplementedError):
        fly_amd.FlatBlockButterflySparsityConfig(6, 1)
    with pytest.raises(NotImplementedError):
        fly_amd.FlatBlockButterflySparsityConfig(8, 4)


def test_index_tables_bit_exact():
    layout = _layout(3, 5, 4, 1)
    layout[1, 3, :] = 0
    layout[2, :, 1] = 0
    assert torch.equal(bu.sdd_table(layout), ob.sdd_lut(layout))
    for by_rows in (True, False):
        for got, want in zip(bu.segment_table(layout, by_rows), ob.segment_table(layout, by_rows)):
            assert got.dtype == torch.int32 and torch.equal(got, want)
    ptr, blk, col, max_nnz = bu.row_table(layout)
    lut, want_max, _, _ = ob.row_lut(layout, 16)
    n_seg = 15
    assert max_nnz == want_max
    assert (ptr[1:] - ptr[:-1]).tolist() == lut[:2 * n_seg].view(n_seg, 2)[:, 0].tolist()
    core = lut[2 * n_seg:].view(-1, 4)
    assert torch.equal(blk, core[:, 0]) and torch.equal(col, core[:, 1])
    # 2-D layout means one head
    assert torch.equal(bu.sdd_table(layout[0]), ob.sdd_lut(layout[0]))


def test_union_order_longest_lists_first():
    """Per head a permutation of its groups, list lengths non-increasing, ties in index order."""
    for H, p, r, seed in ((2, 8, 6, 1), (3, 5, 9, 2), (1, 2, 3, 3)):
        layout = _layout(H, p, r, seed)
        layout[0, 0, :] = 1                                  # a block-row of global tokens
        ptr, _, _ = bu.union_table(layout, rows_per_group=2)
        order = bu.union_order(ptr, H)
        G = (p + 1) // 2
        assert order.dtype == torch.int32 and order.shape == (H * G,)
        counts = (ptr[1:] - ptr[:-1]).reshape(H, G).tolist()
        for h in range(H):
            o = order[h * G:(h + 1) * G].tolist()
            assert sorted(o) == list(range(G))
            assert o == sorted(range(G), key=lambda g: (-counts[h][g], g))
        assert order[0] == 0                                 # the global row's group has every column


def test_union_table_against_loops():
    """Union of block-columns over groups of four block-rows, checked against explicit loops."""
    for H, p, r, seed in ((2, 7, 5, 4), (1, 4, 9, 5), (3, 1, 3, 6)):
        layout = _layout(H, p, r, seed)
        if p > 5:
            layout[0, 4:8, :] = 0                           # an empty group
            layout[1, 1, :] = 0                             # an empty row inside a group
        ids = {}
        for n, (h, i, j) in enumerate(layout.nonzero().tolist()):
            ids[(h, i, j)] = n
        ptr, inner, blk = bu.union_table(layout)
        assert ptr.dtype == inner.dtype == blk.dtype == torch.int32
        G = (p + 3) // 4
        assert ptr.numel() == H * G + 1 and blk.shape == (inner.numel(), 4)
        want_ptr, want_inner, want_blk = [0], [], []
        for h in range(H):
            for gi in range(G):
                for j in range(r):
                    row = [ids.get((h, 4 * gi + w, j), -1) for w in range(4)]
                    if max(row) >= 0:
                        want_inner.append(j)
                        want_blk.append(row)
                want_ptr.append(len(want_inner))
        assert ptr.tolist() == want_ptr and inner.tolist() == want_inner and blk.tolist() == want_blk
        # every block appears exactly once
        assert sorted(x for x in blk.reshape(-1).tolist() if x >= 0) == list(range(int(layout.sum())))


def test_format_helpers_bit_exact():
    layout = _layout(2, 3, 4, 2)
    g = torch.Generator().manual_seed(0)
    x = torch.randn(3, 2, 3 * 8, 4 * 4, generator=g)
    sp = bu.sparsify_tensor(x, layout)
    assert torch.equal(sp, ob.sparsify_tensor(x, layout))
    assert torch.equal(bu.densify_tensor(sp, layout, value=2.0), ob.densify_tensor(sp, layout, value=2.0))
    assert torch.equal(bu.mask_tensor(x, layout, value=-1.0), ob.mask_tensor(x, layout, value=-1.0))
    rows = torch.randn(3, 2, 24, generator=g)
    assert torch.equal(bu.sparsify_broadcast_tensor(rows, layout, 8), ob.sparsify_broadcast_tensor(rows, layout, 8))


def test_masks_and_padding():
    lengths = torch.tensor([3, 0, 5])
    m = fly_amd.LengthMask(lengths, max_len=5)
    assert m.bool_matrix.tolist() == [[1, 1, 1, 0, 0], [0] * 5, [1] * 5]
    assert not m.all_ones and torch.equal(m.lengths, lengths)
    assert torch.equal(m.additive_matrix_finite[0], torch.tensor([0.0, 0.0, 0.0, -1e24, -1e24]))
    assert m.additive_matrix[0, 3] == float('-inf')
    full = fly_amd.FullMask(m.bool_matrix)
    assert torch.equal(full.lengths, lengths)
    with pytest.raises(ValueError, match='not a length mask'):
        fly_amd.FullMask(torch.tensor([[True, False, True]])).lengths
    with pytest.raises(ValueError):
        fly_amd.FullMask(torch.ones(2, 2))
    assert fly_amd.FullMask(4).all_ones and fly_amd.FullMask(2, 3).shape == (2, 3)
    tri = fly_amd.TriangularCausalMask(4)
    assert tri.lower_triangular and tri.bool_matrix.tolist() == torch.ones(4, 4).tril().bool().tolist()
    from fly_amd.masking import pad_mask
    from fly_amd.padding import pad_to_multiple
    assert pad_mask(m, 3, left=False, value=False).bool_matrix.shape == (3, 8)
    assert pad_mask(full, 2, left=False, value=False).bool_matrix[2].tolist() == [1] * 5 + [0, 0]
    x = torch.ones(2, 5, 3, 7)
    y = pad_to_multiple(x, 4, dims=(1, 3))
    assert y.shape == (2, 8, 3, 8) and float(y.sum()) == float(x.sum())
    assert pad_to_multiple(x, 1, dims=-1) is x


def test_matmul_validation_mirrors_reference():
    layout = _layout(2, 2, 3, 3)
    with pytest.raises(NotImplementedError):
        fly_amd.matmul(layout, 16, 'ssd')
    op = fly_amd.matmul(layout, 16, 'dsd')
    assert op.sparse_shape == (int(layout.sum()), 16, 16) and op.dense_inner_size == 48
    a = torch.zeros(1, int(layout.sum()), 16, 16)
    with pytest.raises(ValueError, match='Only GPU devices'):       # blocksparse_matmul.py:682-683
        op(a, torch.zeros(1, 2, 48, 8))
    with pytest.raises(ValueError, match='same dtype'):
        op._validate_inputs(a.cuda() if torch.cuda.is_available() else _fake_cuda(a),
                            _fake_cuda(torch.zeros(1, 2, 48, 8, dtype=torch.float64)))
    dds = fly_amd.matmul(layout, 16, 'dds', trans_b=True)
    assert dds.dense_inner_size == 48 and dds.dense_inner_dim == -1
    assert fly_amd.matmul(layout[0], 16, 'sdd').spdims == (1, 2, 3)


class _FakeCuda(torch.Tensor):
    """A CPU tensor that claims to live on the GPU: lets the shape/dtype validation run here."""
    @property
    def is_cuda(self):
        return True


def _fake_cuda(t):
    return t.as_subclass(_FakeCuda)


def test_matmul_shape_errors_before_launch():
    layout = _layout(2, 2, 3, 3)
    op = fly_amd.matmul(layout, 16, 'dsd')
    nnz = int(layout.sum())
    with pytest.raises(ValueError, match='Expected tensor B to have size 48'):
        op._validate_inputs(_fake_cuda(torch.zeros(1, nnz, 16, 16)), _fake_cuda(torch.zeros(1, 2, 32, 8)))
    with pytest.raises(ValueError, match='trailing dimensions'):
        op._validate_inputs(_fake_cuda(torch.zeros(1, nnz + 1, 16, 16)), _fake_cuda(torch.zeros(1, 2, 48, 8)))
    with pytest.raises(ValueError, match='more than 4 dimensions'):
        op._validate_inputs(_fake_cuda(torch.zeros(1, 1, nnz, 16, 16)), _fake_cuda(torch.zeros(1, 2, 48, 8)))


def test_sblocal_module_interface_and_refusals():
    torch.manual_seed(0)
    attn = fly_amd.SBLocalAttention(local_context=8, dim_heads=16, nb_features=10)
    assert attn.feature_map.projection_matrix.shape == (5, 16)          # buffer name kept for state dicts
    assert 'feature_map.projection_matrix' in attn.state_dict()
    attn.feature_map.new_feature_map('cpu')
    P = attn.feature_map.projection_matrix.clone()
    attn.feature_map.new_feature_map('cpu')                             # drawn once only
    assert torch.equal(P, attn.feature_map.projection_matrix) and float(P.abs().sum()) > 0
    q = torch.zeros(1, 4, 1, 16)
    with pytest.raises(ValueError, match='GPU'):                         # no CPU implementation is shipped
        attn(q, q, q)
    attn.max_weight_elements = 15                                        # the dense matrix is for small problems
    with pytest.raises(NotImplementedError, match='materialises'):
        attn(q, q, q, need_weights=True)
    with pytest.raises(NotImplementedError):
        fly_amd.SBLocalAttention(8, 16, causal=True)(q, q, q)
    with pytest.raises(NotImplementedError):
        fly_amd.SBLocalAttention(8, 16, softmax_eps=1e-3)(q, q, q)
    default = fly_amd.SBLocalAttention(8, 64)
    assert default.feature_map.n_features == int(64 * torch.log(torch.tensor(64.0)))   # feature_maps_sb.py:111


def test_projection_matrix_is_seed_reproducible_and_orthogonal():
    torch.manual_seed(7)
    a = fly_amd.gaussian_orthogonal_random_matrix(96, 64)
    torch.manual_seed(7)
    b = fly_amd.gaussian_orthogonal_random_matrix(96, 64)
    assert torch.equal(a, b) and a.shape == (96, 64)
    unit = a / a.norm(dim=1, keepdim=True)
    assert torch.allclose(unit[:64] @ unit[:64].t(), torch.eye(64), atol=1e-5)
    assert torch.allclose(unit[64:] @ unit[64:].t(), torch.eye(32), atol=1e-5)


def test_blocksparse_linear_init_and_dense_backend():
    """Init statistics and the 'dense' backend (a library GEMM on the densified weight, the
    reference's own backend option, blocksparse_linear.py:163-166) against the oracle."""
    torch.manual_seed(0)
    cfg = fly_amd.FlatBlockButterflySparsityConfig(8, 2, block=32)
    lin = fly_amd.BlockSparseLinear(497, 698, cfg, backend='dense')
    assert lin.layout.shape == (22, 16) and lin.weight.shape == (int(lin.layout.sum()), 32, 32)
    assert lin.nnz_blocks == int(lin.layout.sum()) and 0 < lin.saving < 1
    tri = fly_amd.BlockSparseLinear(497, 698, cfg)
    assert tri.weight.shape == (1, tri.nnz_blocks, 32, 32)               # parameter shape of the GPU backend
    # Kaiming-uniform(a=sqrt5) on the dense matrix scaled by sqrt(ncol/nnz cols): bound = sqrt(1/nnz_in)
    nnz_cols = lin.layout.sum(-1).float() * 32
    bound = (1.0 / nnz_cols).sqrt().max()
    assert float(lin.weight.detach().abs().max()) <= float(bound) + 1e-6
    assert float(lin.bias.abs().max()) <= 1 / (512 ** 0.5) + 1e-6
    x = torch.randn(3, 5, 497)
    ref = ob.blocksparse_linear(x, lin.weight.detach(), lin.layout, 32, lin.bias.detach(), 698)
    assert torch.allclose(lin(x), ref, atol=1e-5)
    with pytest.raises(NotImplementedError):
        tri(x)                                                           # GPU backend refuses CPU tensors
    with pytest.raises(ImportError):
        fly_amd.BlockSparseLinear(64, 64, cfg, backend='huggingface')
    low = fly_amd.LowRank(64, 128, rank=0.25)
    assert low.rank == 16 and low.lr_weight1.shape == (16, 64) and low.lr_weight2.shape == (128, 16)
    svd = fly_amd.LowRank(64, 128, rank=8, init='svd', bias=False)
    assert svd.lr_weight1.shape == (8, 64)
    slr = fly_amd.SparseLRLinear(256, 512, {'_target_': 'src.models.layers.blocksparse_linear.BlockSparseLinear',
                                            'sparsity_config': cfg, 'backend': 'dense'}, rank=16)
    assert set(k for k, _ in slr.named_parameters()) == {
        'bias', 'sparse.weight', 'low_rank.lr_weight1', 'low_rank.lr_weight2', 'gate.weight', 'gate.bias'}
    y = slr(torch.randn(10, 256))
    assert y.shape == (10, 512)


def test_sbblocksparse_module_interface_and_refusals():
    """Constructor / buffers of the block-sparse Scatterbrain layer and what it refuses before any launch
    (the reference asserts masks away, sbblocksparse_attention.py:181; its causal path is unchecked, :147)."""
    cfg = fly_amd.FlatBlockButterflySparsityConfig(4, 2, block=16)
    layer = fly_amd.SBBlockSparseAttention(cfg, dim_heads=32, nb_features=32, max_seq_length=256)
    assert tuple(layer.master_layout.shape) == (16, 16)           # a 2-D layout means one head
    assert tuple(layer.feature_map.projection_matrix.shape) == (16, 32)
    assert tuple(layer.get_layout(64).shape) == (1, 4, 4)
    with pytest.raises(NotImplementedError):
        fly_amd.SBBlockSparseAttention(cfg, dim_heads=32, causal=True)
    q = torch.zeros(1, 40, 1, 32)
    with pytest.raises(ValueError, match='divisible by block size'):
        layer(q, q, q)
    q = torch.zeros(1, 64, 1, 32)
    with pytest.raises(NotImplementedError):
        layer(q, q, q, key_padding_mask=fly_amd.LengthMask(torch.tensor([64]), max_len=64))
    with pytest.raises(ValueError, match='head dim'):
        layer(torch.zeros(1, 64, 1, 16), q, q)


def test_scratch_cache_is_bounded_and_tracks_the_projection_object():
    """The per-module cache of Scatterbrain-local attention: at most max_plans plans, least recently used dropped
    first; the padded projection is remade when the caller's tensor is REPLACED by another of the same shape (same
    version counter, possibly the same address) or written to; copies and pickles of the cache start empty."""
    import copy
    import pickle
    from fly_amd.sblocal_attention import ScratchCache, _padded_projection
    cache = ScratchCache(max_plans=3)
    made = []

    def maker(tag):
        def make():
            made.append(tag)
            return tag
        return make
    for tag in 'abc':
        assert cache.plan(tag, maker(tag)) == tag
    assert cache.plan('a', maker('a')) == 'a' and made == ['a', 'b', 'c']       # hit: nothing made, 'a' now most recent
    cache.plan('d', maker('d'))                                                 # evicts 'b', the least recently used
    assert len(cache) == 3 and set(cache.plans) == {'a', 'c', 'd'}
    cache.plan('b', maker('b'))
    assert made == ['a', 'b', 'c', 'd', 'b'] and set(cache.plans) == {'a', 'd', 'b'}

    P1 = torch.randn(13, 21)
    pad1 = _padded_projection(P1, 16, 32, cache)
    assert pad1.shape == (16, 32) and torch.equal(pad1[:13, :21], P1) and float(pad1[13:].abs().sum()) == 0
    assert _padded_projection(P1, 16, 32, cache) is pad1                        # unchanged tensor: the kept copy
    P2 = torch.randn(13, 21)                                                    # a replacement: same shape, version 0
    assert P2._version == P1._version
    pad2 = _padded_projection(P2, 16, 32, cache)
    assert torch.equal(pad2[:13, :21], P2)
    P2.mul_(2.0)                                                                # written to in place
    assert torch.equal(_padded_projection(P2, 16, 32, cache)[:13, :21], P2)
    exact = torch.randn(16, 32)
    assert _padded_projection(exact, 16, 32, cache) is exact                    # already in kernel form: used as is
    assert len(copy.deepcopy(cache)) == 0 and len(pickle.loads(pickle.dumps(cache))) == 0
    mod = fly_amd.SBLocalAttention(8, dim_heads=16, nb_features=8)
    mod._scratch_cache.plan('x', maker('x'))
    assert len(copy.deepcopy(mod)._scratch_cache) == 0


@pytest.mark.parametrize('block', [16, 32])
def test_tile_mask_table_against_loops(block):
    """The support table of the fused Scatterbrain kernels (per 64-query tile its 32-key tiles, per entry and group of
    16 queries which halves of the tile are on the support) against explicit loops over the layout."""
    from fly_amd.blocksparse_utils import tile_mask_table
    g = torch.Generator().manual_seed(block)
    H, p, r = 3, 11 if block == 16 else 5, 9 if block == 16 else 7
    layout = (torch.rand(H, p, r, generator=g) < 0.35).long()
    layout[1, 2, :] = 0
    ptr, inner, mask = tile_mask_table(layout, block)
    rows, cols = p * block, r * block
    n_qt, n_kt = (rows + 63) // 64, (cols + 31) // 32
    assert ptr.shape == (H * n_qt + 1,) and ptr.dtype == inner.dtype == mask.dtype == torch.int32
    want = []
    for h in range(H):
        for qt in range(n_qt):
            for kt in range(n_kt):
                m4 = []
                for w in range(4):
                    bits = 0
                    for half in range(2):
                        i, j = 64 * qt + 16 * w, 32 * kt + 16 * half
                        if i < rows and j < cols and layout[h, i // block, j // block]:
                            bits |= 1 << half
                    m4.append(bits)
                if any(m4):
                    want.append((h * n_qt + qt, kt, m4))
    assert int(ptr[-1]) == len(want) == inner.numel() and mask.shape == (len(want), 4)
    at = 0
    for grp in range(H * n_qt):
        mine = [e for e in want if e[0] == grp]
        assert int(ptr[grp + 1]) - int(ptr[grp]) == len(mine)
        for e in mine:
            assert int(inner[at]) == e[1] and mask[at].tolist() == e[2]
            at += 1
    # transposed: the table of the transposed layout (64-key tiles against 32-query tiles, the backward's key-major pass)
    for a_, b_ in zip(tile_mask_table(layout, block, transposed=True), tile_mask_table(layout.transpose(1, 2).contiguous(), block)):
        assert torch.equal(a_, b_)
    with pytest.raises(ValueError):
        tile_mask_table(layout, 64)
