"""The block-sparse storage format (src/models/attention/blocksparse_utils.py:8-74) and the index
tables the HIP kernels walk.

A sparse tensor is (..., nnz, blk, blk1): block n is the n-th nonzero of ``layout.flatten()`` for a
layout (H, rows/blk, cols/blk1), i.e. nonzero blocks in (head, block-row, block-col) row-major
order, each stored row-major.
"""
import torch


def _as_layout3(layout):
    layout = torch.as_tensor(layout)
    if layout.ndim == 2:
        layout = layout.unsqueeze(0)
    if layout.ndim != 3:
        raise ValueError('layout must be a 2- or 3-dimensional tensor of 0s and 1s')
    return layout


def sparsify_tensor(x, mask):
    """x (..., H, T, S), mask (H, T/blk, S/blk1) -> (..., nnz, blk, blk1)   (:8-19)."""
    H, p, r = mask.shape
    blk, blk1 = x.shape[-2] // p, x.shape[-1] // r
    lead = x.shape[:-3]
    blocks = x.reshape(*lead, H, p, blk, r, blk1).transpose(-3, -2).reshape(*lead, H * p * r, blk, blk1)
    return blocks[..., mask.flatten().bool().to(x.device), :, :]


def densify_tensor(x, mask, value=0.0):
    """x (..., nnz, blk, blk1), mask (H, p, r) -> (..., H, p*blk, r*blk1), `value` elsewhere (:22-40)."""
    mask = mask.bool().to(x.device)
    lead = x.shape[:-3]
    nnz, blk, blk1 = x.shape[-3:]
    H, p, r = mask.shape
    assert nnz == mask.sum(), 'Mask has a different number of nonzero blocks than input'
    dense = torch.full((*lead, H * p * r, blk, blk1), value, dtype=x.dtype, device=x.device)
    dense[..., mask.flatten(), :, :] = x
    return dense.reshape(*lead, H, p, r, blk, blk1).transpose(-3, -2).reshape(*lead, H, p * blk, r * blk1)


def mask_tensor(x, mask, value=0.0):
    """Keep the nonzero blocks of x (..., H, T, S), set the others to `value` (:45-57)."""
    H, p, r = mask.shape
    blk, blk1 = x.shape[-2] // p, x.shape[-1] // r
    keep = mask.bool().to(x.device).repeat_interleave(blk, dim=1).repeat_interleave(blk1, dim=2)
    return x.masked_fill(~keep, value)


def sparsify_broadcast_tensor(x, mask, block=None):
    """x (B, H, T) -> (B, nnz, blk, 1): for every nonzero block the slice of x for its rows (:60-74).
    `block` is accepted and ignored: the reference's callers pass it although the reference
    function takes two arguments (sbblocksparse_attention.py:197,199)."""
    mask = _as_layout3(mask)
    blk = x.shape[-1] // mask.shape[-2]
    rows = x.reshape(x.shape[0], x.shape[1], mask.shape[-2], blk, 1)
    h_idx, row_idx, _ = torch.nonzero(mask, as_tuple=True)
    return rows[:, h_idx.to(x.device), row_idx.to(x.device)]


# -----------------------------------------------------------------------------------------
# index tables (host side, int32) -- the information of the reference's look-up tables
# (blocksparse_matmul.py:261-276, 356-441; blocksparse_logsumexp.py:107-128) in the CSR-like
# form the HIP kernels consume
# -----------------------------------------------------------------------------------------
def sdd_table(layout):
    """int32 (nnz, 4): (head, block_row, block_col, block_id) per nonzero block, storage order."""
    layout = _as_layout3(layout).cpu()
    nz = layout.nonzero(as_tuple=False)
    ids = torch.arange(nz.shape[0], dtype=nz.dtype).unsqueeze(1)
    return torch.cat([nz, ids], dim=1).to(torch.int32).contiguous()


def segment_table(layout, by_rows):
    """Reduction lists per (head, block-row) [by_rows] or (head, block-col): returns
    (seg_ptr int32 (n_seg+1), seg_blk int32 (nnz) block ids, seg_inner int32 (nnz) the block index
    along the other axis), blocks of a segment in increasing inner index."""
    layout = _as_layout3(layout).cpu().long()
    H, p, r = layout.shape
    nz = layout.nonzero(as_tuple=False)                      # storage order: (h, row, col)
    ids = torch.arange(nz.shape[0])
    if by_rows:
        seg = nz[:, 0] * p + nz[:, 1]
        inner = nz[:, 2]
        n_seg = H * p
    else:
        key = (nz[:, 0] * r + nz[:, 2]) * p + nz[:, 1]       # sort by (h, col, row)
        order = torch.argsort(key, stable=True)
        nz, ids = nz[order], ids[order]
        seg = nz[:, 0] * r + nz[:, 2]
        inner = nz[:, 1]
        n_seg = H * r
    counts = torch.bincount(seg, minlength=n_seg)
    ptr = torch.zeros(n_seg + 1, dtype=torch.int64)
    ptr[1:] = torch.cumsum(counts, 0)
    return ptr.to(torch.int32), ids.to(torch.int32).contiguous(), inner.to(torch.int32).contiguous()


def row_table(layout):
    """Per (head, block-row): (row_ptr, row_blk, row_col, max_row_nnz) for the row operations."""
    ptr, blk, col = segment_table(layout, by_rows=True)
    counts = ptr[1:] - ptr[:-1]
    return ptr, blk, col, int(counts.max()) if counts.numel() else 0


def union_table(layout, rows_per_group=4, transposed=False):
    """Union of block-columns over groups of `rows_per_group` consecutive block-rows of a head
    (ceil(rows / rows_per_group) groups per head, head-major): returns (uni_ptr int32 (n_groups+1),
    uni_inner int32 (n_union) block-columns in increasing order per group, uni_blk int32
    (n_union, rows_per_group) the block id at (row rows_per_group*g + w, that column) or -1).
    transposed=True: the same with the roles of rows and columns exchanged (groups of block-columns,
    unions of their block-rows), block ids still those of the layout's own storage order."""
    layout = _as_layout3(layout).cpu().long()
    ids = (torch.cumsum(layout.reshape(-1), 0) - 1).reshape(layout.shape)
    ids = torch.where(layout > 0, ids, torch.full_like(ids, -1))
    if transposed:
        layout, ids = layout.transpose(1, 2), ids.transpose(1, 2)
    H, p, r = layout.shape
    R = rows_per_group
    G = (p + R - 1) // R
    pad = torch.full((H, G * R - p, r), -1, dtype=ids.dtype)
    ids = torch.cat([ids, pad], dim=1).reshape(H, G, R, r)
    nz = (ids >= 0).any(dim=2).nonzero(as_tuple=False)              # (h, g, col), sorted
    blk = ids[nz[:, 0], nz[:, 1], :, nz[:, 2]]                      # (n_union, R)
    counts = torch.bincount(nz[:, 0] * G + nz[:, 1], minlength=H * G)
    ptr = torch.zeros(H * G + 1, dtype=torch.int64)
    ptr[1:] = torch.cumsum(counts, 0)
    return ptr.to(torch.int32), nz[:, 2].to(torch.int32).contiguous(), blk.to(torch.int32).contiguous()


def tile_mask_table(layout, block, transposed=False):
    """The support of a layout of 16 x 16 or 32 x 32 blocks as the fused Scatterbrain kernels walk it: per (head,
    64-query tile) the 32-key tiles that hold a block of any of the tile's block-rows, and per entry four masks, one per
    group of 16 queries (16 w .. 16 w + 15 of the tile): bit 0 / bit 1 = that group sees keys 0..15 / 16..31 of the
    entry's key tile.  Returns (ptr int32 (H * ceil(rows / 64) + 1), inner int32 (n) key tiles in increasing order per
    query tile, mask int32 (n, 4)); rows and columns past the layout's end count as absent.  transposed: the same with
    the roles of queries and keys exchanged (64-key tiles against 32-query tiles: the key-major pass of the backward)."""
    if block not in (16, 32):
        raise ValueError(f'block size {block}: the fused kernels walk supports of 16 x 16 or 32 x 32 blocks')
    fine = _as_layout3(layout).cpu() > 0
    if transposed:
        fine = fine.transpose(1, 2)
    rep = block // 16
    if rep > 1:
        fine = fine.repeat_interleave(rep, dim=1).repeat_interleave(rep, dim=2)
    H, p16, r16 = fine.shape
    G, C = (p16 + 3) // 4, (r16 + 1) // 2
    padded = torch.zeros(H, 4 * G, 2 * C, dtype=torch.bool)
    padded[:, :p16, :r16] = fine
    halves = padded.view(H, G, 4, C, 2).long()
    mask = (halves[..., 0] + 2 * halves[..., 1]).permute(0, 1, 3, 2)           # (H, G, C, 4)
    nz = (mask > 0).any(dim=3).nonzero(as_tuple=False)                        # (h, g, c), sorted
    counts = torch.bincount(nz[:, 0] * G + nz[:, 1], minlength=H * G)
    ptr = torch.zeros(H * G + 1, dtype=torch.int64)
    ptr[1:] = torch.cumsum(counts, 0)
    return (ptr.to(torch.int32), nz[:, 2].to(torch.int32).contiguous(),
            mask[nz[:, 0], nz[:, 1], nz[:, 2]].to(torch.int32).contiguous())


def union_order(uni_ptr, n_heads):
    """Per head, its groups of union_table sorted by the length of their lists, longest first (ties in
    index order): int32 (n_heads * groups_per_head), entries are group indices within the head."""
    counts = (uni_ptr[1:] - uni_ptr[:-1]).cpu().long().reshape(n_heads, -1)
    return torch.argsort(counts, dim=1, descending=True, stable=True).to(torch.int32).reshape(-1).contiguous()


def union_heavy(uni_ptr, uni_blk, n_heavy_min=32, entries_per_part=12, max_parts=16):
    """The groups of union_table whose lists are long enough to be walked in parts: returns (heavy int32
    (n_heavy) global group indices head * groups + group, parts) with parts = longest list //
    entries_per_part clipped to [2, max_parts]; (empty, 1) when no list has n_heavy_min entries.  A group
    qualifies only if every one of its rows that has any entry in the table's padding sense -- i.e. each of
    its block-rows -- owns at least one block (a part cannot know whether another part saw a block)."""
    ptr = uni_ptr.cpu().long()
    blk = uni_blk.cpu()
    counts = ptr[1:] - ptr[:-1]
    heavy = []
    for gidx in (counts >= n_heavy_min).nonzero().flatten().tolist():
        rows = blk[ptr[gidx]:ptr[gidx + 1]]
        if bool((rows >= 0).any(dim=0).all()):
            heavy.append(gidx)
    if not heavy:
        return torch.zeros(0, dtype=torch.int32), 1
    longest = int(counts[heavy].max())
    return torch.tensor(heavy, dtype=torch.int32), max(2, min(max_parts, longest // entries_per_part))


def group_table(layout, by_rows, max_group=4):
    """Groups of up to `max_group` consecutive segments (of one head) whose reduction lists visit the
    same inner blocks: returns (grp_row0 int32, grp_n int32).  Every segment belongs to one group."""
    layout = _as_layout3(layout).cpu().long()
    if not by_rows:
        layout = layout.transpose(1, 2)
    H, p, _ = layout.shape
    row0, count = [], []
    for h in range(H):
        i = 0
        while i < p:
            n = 1
            while n < max_group and i + n < p and torch.equal(layout[h, i + n], layout[h, i]):
                n += 1
            row0.append(h * p + i)
            count.append(n)
            i += n
    return torch.tensor(row0, dtype=torch.int32), torch.tensor(count, dtype=torch.int32)
