"""Oracle (test infrastructure) for the block-sparse format, matmuls, row ops and layouts.

Follows ``src/models/attention/blocksparse_utils.py``, ``blocksparse_matmul.py`` (the
semantics of SDD / DSD / DDS and the look-up tables), ``blocksparse_logsumexp.py``,
``blocksparse_sum.py``, ``blocksparse_attention.py`` and
``src/models/layers/blocksparse_linear.py`` + ``src/ops/butterfly_factor.py``.

Pinning (tests/test_oracle_blocksparse.py): the format helpers against per-block Python
loops; the matmuls against ``torch.matmul`` on densified operands (what the reference's
test_blocksparse_attention.py:58-80 asserts); the block softmax against ``torch.softmax`` on
a -inf filled dense matrix with empty rows -> 0 (same test); the layouts against the closed
form ``j in {i} U {i xor 2^k}`` and the known block counts; the look-up tables against
brute-force enumeration of ``layout.nonzero()``.
"""
import math

import numpy as np
import torch


# --------------------------------------------------------------------------------------
# storage format -- blocksparse_utils.py:8-74
# --------------------------------------------------------------------------------------
def sparsify_tensor(x, mask):
    """blocksparse_utils.py:8-19.  x (..., H, T, S), mask (H, T/blk, S/blk1) ->
    (..., nnz, blk, blk1); block n is the n-th nonzero of mask.flatten()."""
    H, p, r = mask.shape
    blk, blk1 = x.shape[-2] // p, x.shape[-1] // r
    lead = x.shape[:-3]
    xr = x.reshape(*lead, H, p, blk, r, blk1).movedim(-2, -3)       # ..., H, p, r, blk, blk1
    xr = xr.reshape(*lead, H * p * r, blk, blk1)
    return xr[..., mask.flatten().bool(), :, :]


def densify_tensor(x, mask, value=0.0):
    """blocksparse_utils.py:22-40.  x (..., nnz, blk, blk1) -> (..., H, p*blk, r*blk1)."""
    mask = mask.bool()
    H, p, r = mask.shape
    lead = x.shape[:-3]
    nnz, blk, blk1 = x.shape[-3:]
    assert nnz == int(mask.sum())
    dense = torch.full((*lead, H * p * r, blk, blk1), value, dtype=x.dtype)
    dense[..., mask.flatten(), :, :] = x
    dense = dense.reshape(*lead, H, p, r, blk, blk1).movedim(-2, -3)
    return dense.reshape(*lead, H, p * blk, r * blk1)


def mask_tensor(x, mask, value=0.0):
    """blocksparse_utils.py:45-57: keep the nonzero blocks, fill the others with value."""
    H, p, r = mask.shape
    blk, blk1 = x.shape[-2] // p, x.shape[-1] // r
    keep = mask.bool().repeat_interleave(blk, 1).repeat_interleave(blk1, 2)
    return torch.where(keep, x, torch.full((), value, dtype=x.dtype))


def sparsify_broadcast_tensor(x, mask, block=None):
    """blocksparse_utils.py:60-74.  x (B, H, T) -> (B, nnz, blk, 1): the row vector of each
    nonzero block.  The ignored third argument absorbs the three-argument calls at
    sbblocksparse_attention.py:197,199 and blocksparse_sum.py:146."""
    blk = x.shape[-1] // mask.shape[-2]
    xr = x.reshape(x.shape[0], x.shape[1], mask.shape[-2], blk, 1)
    h_idx, row_idx, _ = torch.nonzero(mask, as_tuple=True)
    return xr[:, h_idx, row_idx]


# --------------------------------------------------------------------------------------
# matmuls -- semantics of blocksparse_matmul.py:279-346 (SDD), :444-488 (DDS), :491-535 (DSD)
# --------------------------------------------------------------------------------------
def _layout3(layout):
    layout = torch.as_tensor(layout)
    return (layout.unsqueeze(0) if layout.ndim == 2 else layout).long()     # :649-652


def sdd(a, b, layout, block, trans_a=False, trans_b=False):
    """SDD: sparsify(op(a) @ op(b)) -- what test_blocksparse_attention.py:79 asserts.
    a, b (B,H,.,.) dense; returns (B, nnz, blk, blk) in the input dtype with fp32+ math."""
    layout = _layout3(layout)
    A = a.transpose(-1, -2) if trans_a else a
    Bm = b.transpose(-1, -2) if trans_b else b
    acc = torch.float64 if a.dtype == torch.float64 else torch.float32
    c = A.to(acc) @ Bm.to(acc)
    return sparsify_tensor(c, layout).to(a.dtype)


def dsd(a_sp, b, layout, block, trans_a=False, trans_b=False):
    """DSD: op(densify(a_sp)) @ op(b) -> (B,H,M,N)."""
    layout = _layout3(layout)
    acc = torch.float64 if b.dtype == torch.float64 else torch.float32
    A = densify_tensor(a_sp.to(acc), layout)
    A = A.transpose(-1, -2) if trans_a else A
    Bm = (b.transpose(-1, -2) if trans_b else b).to(acc)
    return (A @ Bm).to(b.dtype)


def dds(a, b_sp, layout, block, trans_a=False, trans_b=False):
    """DDS: op(a) @ op(densify(b_sp)) -> (B,H,M,N)."""
    layout = _layout3(layout)
    acc = torch.float64 if a.dtype == torch.float64 else torch.float32
    Bm = densify_tensor(b_sp.to(acc), layout)
    Bm = Bm.transpose(-1, -2) if trans_b else Bm
    A = (a.transpose(-1, -2) if trans_a else a).to(acc)
    return (A @ Bm).to(a.dtype)


# --------------------------------------------------------------------------------------
# row operations over the nonzero blocks of a block-row
# --------------------------------------------------------------------------------------
def block_softmax(x_sp, layout, block, scale=1.0, key_padding_mask=None, attn_mask=None,
                  key_padding_mask_mode='add', attn_mask_mode='add'):
    """triton.ops.blocksparse.softmax as called at blocksparse_attention.py:146-152 and
    checked at tests/models/attention/test_blocksparse_attention.py:69-80: softmax over the
    nonzero blocks of each row of (x*scale + kpm[b,s] + am[t,s]) in fp32; 'mul' modes map
    0 -> -inf and nonzero -> 0 first.  Rows with no finite entry come out as NaN, as in the
    third-party kernel (the caller applies nan_to_num_); rows of a block-row with no blocks
    do not exist in the sparse tensor.  Returns a new tensor of x's dtype."""
    layout = _layout3(layout)
    dense = densify_tensor(x_sp.float(), layout, value=float('-inf')) * scale
    if key_padding_mask is not None:
        kpm = key_padding_mask.float()
        if key_padding_mask_mode == 'mul':
            kpm = torch.where(kpm == 0, torch.full_like(kpm, float('-inf')), torch.zeros_like(kpm))
        dense = dense + kpm[:, None, None, :]
    if attn_mask is not None:
        am = attn_mask.float()
        if attn_mask_mode == 'mul':
            am = torch.where(am == 0, torch.full_like(am, float('-inf')), torch.zeros_like(am))
        dense = dense + am[None, None, :, :]
    p = torch.softmax(dense, dim=-1)
    return sparsify_tensor(p, layout).to(x_sp.dtype)


def block_logsumexp(x_sp, layout, block):
    """blocksparse_logsumexp.py:29-60,130-147: row logsumexp over nonzero blocks -> (B,H,M);
    rows of empty block-rows stay 0 (output is zero-initialised, :132)."""
    layout = _layout3(layout)
    dense = densify_tensor(x_sp.float(), layout, value=float('-inf'))
    out = torch.logsumexp(dense, dim=-1)
    empty = (layout.sum(-1) == 0).repeat_interleave(block, 1)
    return torch.where(empty.unsqueeze(0), torch.zeros_like(out), out).to(x_sp.dtype)


def block_sum(x_sp, layout, block):
    """blocksparse_sum.py:30-60,123-135: row sum over nonzero blocks -> (B,H,M)."""
    layout = _layout3(layout)
    return densify_tensor(x_sp.float(), layout).sum(-1).to(x_sp.dtype)


# --------------------------------------------------------------------------------------
# look-up tables
# --------------------------------------------------------------------------------------
def sdd_lut(layout):
    """blocksparse_matmul.py:261-276 with start_width=1: libtriton.superblock reduces to one
    int32 row (head, block_row, block_col, block_id) per nonzero block in row-major order
    (pinned by sdd == sparsify_tensor in the reference's test)."""
    layout = _layout3(layout)
    nz = layout.nonzero(as_tuple=False)
    ids = torch.arange(nz.shape[0]).view(-1, 1)
    return torch.cat([nz, ids], 1).to(torch.int32)


def row_lut(layout, block):
    """blocksparse_logsumexp.py:107-128 (also the table of the Triton softmax): header
    (row_nnz, offset) per (head, block-row) with offset = 4*exclusive_cumsum + 2*n_rows, then
    core (block_id, col, row, head) per nonzero block.  Returns (lut int32, max_row_nnz,
    n_head, n_row)."""
    layout = _layout3(layout)
    sizes = layout.sum(-1).flatten()
    offsets = torch.zeros_like(sizes)
    offsets[1:] = torch.cumsum(sizes[:-1], 0)
    nz = layout.nonzero(as_tuple=False)
    idx = torch.arange(nz.shape[0])
    core = torch.stack((idx, nz[:, 2], nz[:, 1], nz[:, 0]), 1).view(-1)
    offsets = offsets * 4 + 2 * sizes.numel()
    header = torch.stack((sizes, offsets), 1).view(-1)
    lut = torch.cat((header, core)).to(torch.int32)
    return lut, int(sizes.max()), layout.shape[0], layout.shape[1] * block


def segment_table(layout, by_rows):
    """The reduction lists a DSD / DDS kernel walks, in the order blocksparse_matmul.py:356-441
    visits them: for every (head, output block index) the (sparse block id, inner block index)
    pairs in increasing inner index.  by_rows=True groups by block-row (DSD, DDS with
    trans_b); False groups by block-column.  Returns (ptr int32 (nseg+1), blk_id int32,
    inner int32)."""
    layout = _layout3(layout).numpy()
    H, p, r = layout.shape
    ids = np.full(layout.shape, -1, dtype=np.int64)
    ids[layout != 0] = np.arange(int((layout != 0).sum()))
    ptr, blk, inner = [0], [], []
    for h in range(H):
        for o in range(p if by_rows else r):
            line = ids[h, o, :] if by_rows else ids[h, :, o]
            for x in np.nonzero(line >= 0)[0]:
                blk.append(line[x])
                inner.append(x)
            ptr.append(len(blk))
    return (torch.tensor(ptr, dtype=torch.int32), torch.tensor(blk, dtype=torch.int32),
            torch.tensor(inner, dtype=torch.int32))


# --------------------------------------------------------------------------------------
# layouts -- src/ops/butterfly_factor.py:8-26, blocksparse_linear.py:175-211
# --------------------------------------------------------------------------------------
def butterfly_factor_to_matrix(twiddle, factor_index):
    """butterfly_factor.py:8-26, restated with explicit loops: the dense matrix of butterfly
    factor `factor_index` (stride b**factor_index) with twiddle (n/b, b, b)."""
    n_div_b, b, _ = twiddle.shape
    n = b * n_div_b
    stride = b ** factor_index
    out = torch.zeros(n, n, dtype=twiddle.dtype)
    tw = twiddle.reshape(n // (b * stride), stride, b, b)            # (diagblk, stride, i, j)
    for d in range(n // (b * stride)):
        for s in range(stride):
            for i in range(b):
                for j in range(b):
                    out[d * b * stride + i * stride + s, d * b * stride + j * stride + s] = \
                        tw[d, s, i, j]
    return out


def flat_butterfly_layout(out_features, in_features, butterfly_size, n_factors, block=32,
                          global_size=0, shuffle=False):
    """FlatBlockButterflySparsityConfig.make_layout, blocksparse_linear.py:191-211."""
    assert out_features % block == 0 and in_features % block == 0
    twiddle = torch.ones(butterfly_size // 2, 2, 2)
    layout = sum(butterfly_factor_to_matrix(twiddle, i) for i in range(n_factors))
    layout = layout.bool().int()
    if shuffle:                                                       # :196-200
        log_n = int(math.log2(butterfly_size))
        ngroups = 2 ** (log_n - n_factors)
        layout = layout.reshape(butterfly_size, ngroups, butterfly_size // ngroups)
        layout = layout.transpose(1, 2).reshape(butterfly_size, butterfly_size)
    f, f1 = out_features // butterfly_size, in_features // butterfly_size
    layout = layout.repeat_interleave(f, 0).repeat_interleave(f1, 1)  # :202-203
    if global_size > 0:                                               # :204-206
        layout[:global_size] = 1
        layout[:, :global_size] = 1
    p, r = out_features // block, in_features // block
    layout = layout.reshape(p, block, r, block).permute(0, 2, 1, 3).reshape(p, r, -1)
    return (layout > 0).any(dim=-1).int()


def band_layout(n_row_blocks, n_col_blocks, half_width):
    """Local band in block units: layout[r, c] = 1 iff |r - c| <= half_width."""
    r = torch.arange(n_row_blocks).view(-1, 1)
    c = torch.arange(n_col_blocks).view(1, -1)
    return ((r - c).abs() <= half_width).int()


# --------------------------------------------------------------------------------------
# BlockSparseAttention.forward -- blocksparse_attention.py:88-166
# --------------------------------------------------------------------------------------
def blocksparse_attention(query, key, value, master_layout, block, softmax_temp=None,
                          key_lengths=None, attn_mask_bool=None):
    """blocksparse_attention.py:88-166 with dropout off.  query (B,T,H,E), key (B,S,H,E),
    value (B,S,H,D); master_layout (H, nb, nb).  Pads to multiples of block on (seq, feature)
    (:107-109), masks padded keys (:117-127), SDD -> softmax -> nan_to_num -> DSD, un-pads."""
    import torch.nn.functional as F
    B, T0, H, E0 = query.shape
    S0, D0 = key.shape[1], value.shape[3]

    def pad(x):
        ps = (-x.shape[1]) % block
        pf = (-x.shape[3]) % block
        return F.pad(x, (0, pf, 0, 0, 0, ps))
    q, k, v = pad(query), pad(key), pad(value)
    T, S = q.shape[1], k.shape[1]
    t = softmax_temp or 1 / math.sqrt(E0)                                          # :114
    kpm = None
    if key_lengths is not None or S > S0:
        lens = key_lengths if key_lengths is not None else torch.full((B,), S0, dtype=torch.long)
        kpm = torch.log((torch.arange(S).view(1, S) < lens.view(B, 1)).float())
    am = None
    if attn_mask_bool is not None:
        am = torch.log(F.pad(attn_mask_bool, (0, S - S0, 0, T - T0), value=False).float())
    q, k, v = (x.permute(0, 2, 1, 3).contiguous() for x in (q, k, v))
    layout = master_layout[:, :T // block, :S // block]
    qk = sdd(q, k, layout, block, trans_b=True)
    p = block_softmax(qk, layout, block, scale=t, key_padding_mask=kpm, attn_mask=am)
    if kpm is not None or am is not None:
        p = p.nan_to_num()
    out = dsd(p, v, layout, block)
    return out.permute(0, 2, 1, 3)[:, :T0, :, :D0]


# --------------------------------------------------------------------------------------
# Pixelfly linear -- blocksparse_linear.py:134-172, fastlinear.py:773-774, 814-827
# --------------------------------------------------------------------------------------
def blocksparse_linear(x, weight_sp, layout, block, bias=None, out_features=None):
    """blocksparse_linear.py:134-172 (any backend; the dense one is :163-166):
    y = x_padded @ densify(W)^T, sliced to out_features, plus bias."""
    import torch.nn.functional as F
    W = densify_tensor(weight_sp.reshape(-1, block, block).float().unsqueeze(0),
                       torch.as_tensor(layout).unsqueeze(0))[0, 0]
    in_ext = W.shape[1]
    if x.shape[-1] < in_ext:
        x = F.pad(x, (0, in_ext - x.shape[-1]))
    y = (x.float() @ W.t()).to(x.dtype)
    if out_features is not None:
        y = y[..., :out_features]
    return y if bias is None else y + bias.to(y.dtype)


def sparse_lr_linear(x, sparse_out, lr_weight1, lr_weight2, gate_weight=None, gate_bias=None,
                     bias=None):
    """fastlinear.py:773-774 and 814-827: lerp(sparse, lowrank, g) + bias with
    g = sigmoid(gate(x)) or 0.5."""
    import torch.nn.functional as F
    low = F.linear(F.linear(x, lr_weight1), lr_weight2)
    g = torch.sigmoid(F.linear(x, gate_weight, gate_bias)) if gate_weight is not None else 0.5
    out = torch.lerp(sparse_out, low, g)
    return out if bias is None else out + bias.to(out.dtype)
