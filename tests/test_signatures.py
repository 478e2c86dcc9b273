"""Drop-in check of the Python surface: the constructor / forward / call signatures of this package's
classes and functions against the reference's, read from the reference's source files as text (parsed
with ``ast``; nothing of the reference is imported or executed).  Every parameter of the reference must
be there under the same name, in the same order, with the same default (a parameter the reference
requires may be optional here); this package may add optional parameters after them.  Skipped where the reference tree is not present (the GPU box)."""
import ast
import inspect
import os

import pytest

REF = '/root/reference/src/models'
pytestmark = pytest.mark.skipif(not os.path.isdir(REF), reason='reference tree not present')

# (reference file, class or None, function, object path in this package)
CASES = [
    ('attention/sblocal_attention.py', 'SBLocalAttention', '__init__', 'SBLocalAttention.__init__'),
    ('attention/sblocal_attention.py', 'SBLocalAttention', 'forward', 'SBLocalAttention.forward'),
    ('attention/local_attention.py', 'LocalAttention', '__init__', 'LocalAttention.__init__'),
    ('attention/local_attention.py', 'LocalAttention', 'forward', 'LocalAttention.forward'),
    ('attention/blocksparse_attention.py', 'BlockSparseAttention', '__init__', 'BlockSparseAttention.__init__'),
    ('attention/blocksparse_attention.py', 'BlockSparseAttention', 'forward', 'BlockSparseAttention.forward'),
    ('attention/sbblocksparse_attention.py', 'SBBlockSparseAttention', '__init__', 'SBBlockSparseAttention.__init__'),
    ('attention/sbblocksparse_attention.py', 'SBBlockSparseAttention', 'forward', 'SBBlockSparseAttention.forward'),
    ('attention/blocksparse_matmul.py', 'matmul', '__init__', 'matmul.__init__'),
    ('attention/blocksparse_matmul.py', 'matmul', '__call__', 'matmul.__call__'),
    ('attention/blocksparse_logsumexp.py', 'logsumexp', '__init__', 'logsumexp.__init__'),
    ('attention/blocksparse_logsumexp.py', 'logsumexp', '__call__', 'logsumexp.__call__'),
    ('attention/blocksparse_sum.py', 'blocksparse_sum', '__init__', 'blocksparse_sum.__init__'),
    ('attention/blocksparse_sum.py', 'blocksparse_sum', '__call__', 'blocksparse_sum.__call__'),
    ('layers/blocksparse_linear.py', 'BlockSparseLinear', '__init__', 'BlockSparseLinear.__init__'),
    ('layers/blocksparse_linear.py', 'BlockSparseLinear', 'forward', 'BlockSparseLinear.forward'),
    ('layers/blocksparse_linear.py', 'FlatBlockButterflySparsityConfig', '__init__',
     'FlatBlockButterflySparsityConfig.__init__'),
    ('layers/blocksparse_linear.py', 'FlatBlockButterflySparsityConfig', 'make_layout',
     'FlatBlockButterflySparsityConfig.make_layout'),
    ('layers/fastlinear.py', 'LowRank', '__init__', 'LowRank.__init__'),
    ('layers/fastlinear.py', 'LowRank', 'forward', 'LowRank.forward'),
    ('layers/fastlinear.py', 'SparseLRLinear', '__init__', 'SparseLRLinear.__init__'),
    ('layers/fastlinear.py', 'SparseLRLinear', 'forward', 'SparseLRLinear.forward'),
    ('attention/feature_maps_sb.py', 'SBPerformerFeatures', '__init__', 'SBPerformerFeatures.__init__'),
    ('attention/feature_maps_sb.py', 'SBPerformerFeatures', 'new_feature_map', 'SBPerformerFeatures.new_feature_map'),
    ('attention/feature_maps_sb.py', 'SBPerformerFeatures', 'forward_queries', 'SBPerformerFeatures.forward_queries'),
    ('attention/feature_maps_sb.py', 'SBPerformerFeatures', 'forward_keys', 'SBPerformerFeatures.forward_keys'),
    ('modules/masking.py', 'FullMask', '__init__', 'FullMask.__init__'),
    ('modules/masking.py', 'LengthMask', '__init__', 'LengthMask.__init__'),
    ('modules/masking.py', 'TriangularCausalMask', '__init__', 'TriangularCausalMask.__init__'),
    ('attention/blocksparse_utils.py', None, 'sparsify_tensor', 'sparsify_tensor'),
    ('attention/blocksparse_utils.py', None, 'densify_tensor', 'densify_tensor'),
    ('attention/blocksparse_utils.py', None, 'mask_tensor', 'mask_tensor'),
    ('attention/blocksparse_utils.py', None, 'sparsify_broadcast_tensor', 'sparsify_broadcast_tensor'),
    ('attention/projection_utils.py', None, 'gaussian_orthogonal_random_matrix', 'gaussian_orthogonal_random_matrix'),
    ('modules/multihead_attention.py', 'MultiheadAttention', '__init__', 'MultiheadAttention.__init__'),
    ('modules/multihead_attention.py', 'MultiheadAttention', 'forward', 'MultiheadAttention.forward'),
    ('modules/multihead_attention.py', 'InProjContainer', '__init__', 'multihead_attention.InProjContainer.__init__'),
    ('modules/multihead_attention.py', 'InProjContainer', 'forward', 'multihead_attention.InProjContainer.forward'),
]


def reference_parameters(path, cls, func):
    """[(name, default source or None)] of a function in a reference file, from its syntax tree."""
    tree = ast.parse(open(os.path.join(REF, path)).read())
    body = tree.body
    if cls is not None:
        body = next(n for n in body if isinstance(n, ast.ClassDef) and n.name == cls).body
    fn = next(n for n in body if isinstance(n, ast.FunctionDef) and n.name == func)
    args = fn.args
    pos = args.posonlyargs + args.args
    defaults = [None] * (len(pos) - len(args.defaults)) + [ast.unparse(d) for d in args.defaults]
    out = list(zip((a.arg for a in pos), defaults))
    out += [(a.arg, None if d is None else ast.unparse(d)) for a, d in zip(args.kwonlyargs, args.kw_defaults)]
    return out, args.vararg is not None, args.kwarg is not None


def same_default(ref_src, value):
    try:
        ref = ast.literal_eval(ref_src)
    except (ValueError, SyntaxError):
        return True          # an expression (e.g. a name): compared by eye in the docstrings, not here
    if isinstance(ref, float) or isinstance(value, float):
        return value is not None and ref is not None and float(ref) == float(value)
    return ref == value


@pytest.mark.parametrize('path,cls,func,mine', CASES, ids=[c[3] for c in CASES])
def test_signature_is_a_superset_of_the_references(path, cls, func, mine):
    import fly_amd
    obj = fly_amd
    for part in mine.split('.'):
        obj = getattr(obj, part)
    ref_params, _, _ = reference_parameters(path, cls, func)
    sig = inspect.signature(obj)
    mine_params = list(sig.parameters.values())
    names = [p.name for p in mine_params]
    assert names[:len(ref_params)] == [n for n, _ in ref_params], (names, ref_params)
    for (name, default), p in zip(ref_params, mine_params):
        if default is not None:
            assert p.default is not inspect.Parameter.empty, f'{name}: default {default} missing'
            assert same_default(default, p.default), f'{name}: default {p.default!r} != reference {default}'
    for p in mine_params[len(ref_params):]:
        assert p.default is not inspect.Parameter.empty or p.kind in (p.VAR_POSITIONAL, p.VAR_KEYWORD), \
            f'extra parameter {p.name} must be optional'
