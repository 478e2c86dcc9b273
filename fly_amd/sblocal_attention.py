"""Scatterbrain-local attention on the HIP kernels: drop-in for
src/models/attention/sblocal_attention.py (class SBLocalAttention, :15-137)."""
import ctypes
import math
import weakref

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import _lib
from .feature_maps_sb import SBPerformerFeatures, softmax_kernel

_HEAD_DIMS = (32, 64, 128)       # padded head dims the kernels are instantiated for
_FEATURE_ROWS = (16, 32, 64, 128)  # padded projection rows (m/2)


def _round_up_choice(n, choices, what):
    for c in choices:
        if n <= c:
            return c
    raise NotImplementedError(f'{what}={n} exceeds the largest supported size {choices[-1]}')


def _vector_ready(x):
    """16-byte vector access needs a unit inner stride, strides in multiples of 4 elements and an
    aligned base pointer."""
    return (x.stride(-1) == 1 and all(s % 4 == 0 for s in x.stride()[:-1])
            and x.data_ptr() % 16 == 0)


class SBLocalPlan:
    """The device scratch and the C-ABI calls for one problem shape.  Callers that run the same shape
    repeatedly (serving loops, benchmarks, the module below) keep one plan and call ``run`` with tensors
    that are already padded and vector-ready; nothing is allocated after the first call.

    q (B,T,H,dim), k, v (B,S,H,dim), proj (mh, dim) float32, lens (B,) int64 or None,
    out (B,T,H,dim), log_norm (B,H,T) float32.  The scratch of one plan is shared by its runs: runs
    of the same plan on different streams race.

    ``run`` is one library call (flyhip_sblocal_forward) on one workspace;
    ``run_keys`` / ``run_queries`` are the two halves as separate calls (flyhip_sb_kv_reduce,
    flyhip_sblocal_fwd) on individually allocated buffers, which are created on first use."""

    def __init__(self, B, H, T, S, dim, mh, mh_valid, dtype, device, local_context, n_parts=None,
                 operand_images=True, exact_fp32=False):
        n_chunks, n_split, parts = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
        _lib.call('flyhip_sb_plan_for', B, H, T, S, local_context, dim, mh, _lib.DTYPE_CODE[dtype],
                  ctypes.byref(n_chunks), ctypes.byref(n_split), ctypes.byref(parts))
        self.n_chunks, self.n_split = n_chunks.value, n_split.value
        self.planned_parts = parts.value
        self.n_parts = parts.value if n_parts is None else n_parts
        self.local_context = local_context
        self.shape = (B, H, T, S, dim, mh, mh_valid)
        self.device = torch.device(device)
        self.dtype = dtype
        self.code = _lib.DTYPE_CODE[dtype]
        self.operand_images = operand_images
        # float inputs only: every product on the fp32 matrix pipe (flag FLYHIP_SB_EXACT_FP32 of the one-call entry
        # point) instead of bf16 pieces on the bf16 pipe
        self.flags = _lib.SB_EXACT_FP32 if (exact_fp32 and dtype == torch.float32) else 0
        self.workspace = None
        self._buffers = False

    def _workspace(self):
        if self.workspace is None:
            B, H, T, S, dim, mh, _ = self.shape
            size = _lib.load().flyhip_sb_workspace_bytes(B, H, T, S, dim, mh, self.local_context, self.code, self.flags)
            if size < 0:
                raise ValueError('flyhip_sb_workspace_bytes rejected the problem shape')
            self.workspace = torch.empty(size, dtype=torch.uint8, device=self.device)
        return self.workspace

    def _make_buffers(self):
        """Scratch of the two-call path, one tensor each."""
        if self._buffers:
            return
        B, H, T, S, dim, mh, _ = self.shape
        dtype, device = self.dtype, self.device
        m, f32 = 2 * mh, torch.float32
        self.kfeat = torch.empty(B, H, self.n_chunks * 64, m, dtype=dtype, device=device)   # opaque, in the input dtype
        self.chunk_scale = torch.empty(B, H, self.n_chunks, dtype=f32, device=device)
        self.kv_part = torch.empty(B, H, self.n_split, m * (dim + 1), dtype=f32, device=device)
        self.part_max = torch.empty(B, H, self.n_split, dtype=f32, device=device)
        self.kv = torch.empty(B, H, m, dim, dtype=f32, device=device)
        self.ksum = torch.empty(B, H, m, dtype=f32, device=device)
        self.kmax = torch.empty(B, H, dtype=f32, device=device)
        self.vt = self.kvt = None
        if dtype == torch.float32 and self.operand_images:
            # float inputs: the band kernel runs on the bf16 matrix pipe from images of every 32-key tile
            # (K in two bf16 pieces, V transposed in three; kfeat then holds the features in two pieces);
            # 128 E + 192 D bytes per tile, two tiles per 64-key chunk.  Without it (block-sparse supports)
            # the fp32-MFMA kernels run from fp32 features.
            self.vt = torch.empty(B, H, self.n_chunks, 2 * (128 * dim + 192 * dim), dtype=torch.uint8, device=device)
        if dtype == torch.bfloat16:
            # bf16 inputs: V per 32-key tile and K'^T V in the operand order of the bf16 MFMA (opaque)
            self.vt = torch.empty(B, H, self.n_chunks * 64, dim, dtype=dtype, device=device)
            self.kvt = torch.empty(B, H, 2, dim, m, dtype=dtype, device=device)     # (two bf16 pieces)
        # with several parts per query tile the key pass also computes the query features, once
        self.part_ws = self.qfeat = self.q_lsq = None
        if self.n_parts > 1:
            self.part_ws = torch.empty(B * H * ((T + 63) // 64) * self.n_parts * 64 * (dim + 5), dtype=f32,
                                       device=device)
            self.qfeat = torch.empty(B, H, T, m, dtype=f32, device=device)
            self.q_lsq = torch.empty(B, H, T, dtype=f32, device=device)
        self._buffers = True

    def run_keys(self, q, k, v, proj, lens, t, stream=None, io_code=0):
        """The key-side pass (features of the keys, K'^T V, sum K'); with several parts per query
        tile also the features of the queries `q`."""
        B, H, T, S, dim, mh, mh_valid = self.shape
        self._make_buffers()
        stream = _lib.stream_ptr(self.device) if stream is None else stream
        q_args = (None, None, None, 0, 0, 0, 0)
        if self.n_parts > 1:
            q_args = (q.data_ptr(), self.qfeat.data_ptr(), self.q_lsq.data_ptr(), T,
                      q.stride(0), q.stride(2), q.stride(1))
        _lib.call('flyhip_sb_kv_reduce', k.data_ptr(), v.data_ptr(), proj.data_ptr(), _lib.ptr(lens),
                  self.kfeat.data_ptr(), self.chunk_scale.data_ptr(), self.kv_part.data_ptr(),
                  self.part_max.data_ptr(), self.kv.data_ptr(), self.ksum.data_ptr(), self.kmax.data_ptr(),
                  *q_args, _lib.ptr(self.vt), _lib.ptr(self.kvt), B, H, S, dim, dim, mh, mh_valid, self.n_split,
                  k.stride(0), k.stride(2), k.stride(1), v.stride(0), v.stride(2), v.stride(1),
                  t, self.code | (io_code << 8), stream)

    def run_queries(self, q, k, v, proj, lens, local_context, t, out, log_norm, stream=None):
        B, H, T, S, dim, mh, mh_valid = self.shape
        self._make_buffers()
        stream = _lib.stream_ptr(self.device) if stream is None else stream
        _lib.call('flyhip_sblocal_fwd', q.data_ptr(), k.data_ptr(), v.data_ptr(), proj.data_ptr(),
                  self.kfeat.data_ptr(), self.chunk_scale.data_ptr(), self.kv.data_ptr(),
                  self.ksum.data_ptr(), self.kmax.data_ptr(), _lib.ptr(self.qfeat), _lib.ptr(self.q_lsq),
                  _lib.ptr(self.vt), _lib.ptr(self.kvt), self.kv_part.data_ptr(), self.part_max.data_ptr(),
                  self.n_split, _lib.ptr(lens), out.data_ptr(), log_norm.data_ptr(), _lib.ptr(self.part_ws), self.n_parts,
                  B, H, T, S, dim, dim, mh, mh_valid, local_context,
                  q.stride(0), q.stride(2), q.stride(1), k.stride(0), k.stride(2), k.stride(1),
                  v.stride(0), v.stride(2), v.stride(1), out.stride(0), out.stride(2), out.stride(1),
                  t, self.code, stream)

    def run_queries_static(self, q, k, v, proj, lens, local_context, t, out, log_norm, stream=None):
        """``run_queries`` through flyhip_sblocal_fwd_static: the partial outputs go to the library's
        built-in scratch array instead of ``self.part_ws`` (nothing is allocated by the call)."""
        B, H, T, S, dim, mh, mh_valid = self.shape
        self._make_buffers()
        stream = _lib.stream_ptr(self.device) if stream is None else stream
        _lib.call('flyhip_sblocal_fwd_static', q.data_ptr(), k.data_ptr(), v.data_ptr(), proj.data_ptr(),
                  self.kfeat.data_ptr(), self.chunk_scale.data_ptr(), self.kv.data_ptr(),
                  self.ksum.data_ptr(), self.kmax.data_ptr(), _lib.ptr(self.qfeat), _lib.ptr(self.q_lsq),
                  _lib.ptr(self.vt), _lib.ptr(self.kvt), self.kv_part.data_ptr(), self.part_max.data_ptr(),
                  self.n_split, _lib.ptr(lens), out.data_ptr(), log_norm.data_ptr(), self.n_parts,
                  B, H, T, S, dim, dim, mh, mh_valid, local_context,
                  q.stride(0), q.stride(2), q.stride(1), k.stride(0), k.stride(2), k.stride(1),
                  v.stride(0), v.stride(2), v.stride(1), out.stride(0), out.stride(2), out.stride(1),
                  t, self.code, stream)

    def run_block_sparse(self, q, k, v, proj, t, tables, out, log_norm, dropout=(0.0, 0), io_code=0):
        """Scatterbrain attention whose exact part lives on a block-sparse support instead of a band: the
        key pass as in ``run``, then the band kernel walking lists of 32-key tiles (``tables`` =
        blocksparse_utils.tile_mask_table(layout, block) on the device) -- on bf16 pieces from the key pass's tile images
        when the plan has them (``operand_images``: float32, head dims up to 64, up to 128 features, no dropout), else on
        the fp32 matrix pipe.  One part per query tile, no key lengths.
        dropout: (probability, seed) of the dropout of the exact weights inside the fp32 kernel.
        io_code: with operand images, q, k, v and out are tensors of that 2-byte element type (_lib.DTYPE_CODE of bfloat16 or
        float16), widened as the kernels load them and rounded as they store: no float32 copies of them."""
        B, H, T, S, dim, mh, mh_valid = self.shape
        self._make_buffers()
        tl_ptr, tl_inner, tl_blk = tables[:3]
        tl_order = tables[3] if len(tables) > 3 else None      # union_order(tl_ptr, H): longest lists first
        # long lists walked in parts (sbblocksparse_attention.fused_tables): scratch for their partials
        tl_heavy, n_heavy, parts = None, 0, 1
        if len(tables) > 5 and tables[4].numel() > 0:
            tl_heavy, n_heavy, parts = tables[4], tables[4].numel(), int(tables[5])
            need = (B * n_heavy * parts * 64 * (dim + 5), B * n_heavy * 64 * 2 * mh)
            if getattr(self, '_heavy_sizes', None) != need:
                self.part_ws = torch.empty(need[0], dtype=torch.float32, device=self.device)
                self.qfeat = torch.empty(need[1], dtype=torch.float32, device=self.device)
                self._heavy_sizes = need
        with torch.cuda.device(self.device):
            stream = _lib.stream_ptr(self.device)
            self.run_keys(q, k, v, proj, None, t, stream, io_code=io_code)
            _lib.call('flyhip_sbblocksparse_fwd', q.data_ptr(), k.data_ptr(), v.data_ptr(), proj.data_ptr(),
                      self.kfeat.data_ptr(), _lib.ptr(self.vt), self.chunk_scale.data_ptr(), self.kv.data_ptr(),
                      self.ksum.data_ptr(), self.kmax.data_ptr(), tl_ptr.data_ptr(), _lib.table_ptr(tl_inner),
                      _lib.table_ptr(tl_blk), _lib.ptr(tl_order), _lib.ptr(tl_heavy), n_heavy, parts,
                      _lib.ptr(self.part_ws) if n_heavy else None, _lib.ptr(self.qfeat) if n_heavy else None,
                      out.data_ptr(), log_norm.data_ptr(),
                      B, H, T, S, dim, dim, mh, mh_valid,
                      q.stride(0), q.stride(2), q.stride(1), k.stride(0), k.stride(2), k.stride(1),
                      v.stride(0), v.stride(2), v.stride(1), out.stride(0), out.stride(2), out.stride(1),
                      t, self.code | (io_code << 8), float(dropout[0]), int(dropout[1]), stream)

    def run(self, q, k, v, proj, lens, local_context, t, out, log_norm, dropout=(0.0, 0), io_code=0):
        """dropout: (probability, seed) -- dropout of the exact weights inside the band kernel (float32 inputs on the
        bf16-piece kernels; the library refuses it elsewhere); the one-call path only.
        io_code: a float32 plan on operand images takes float16 q, k, v and out as they are (_lib.DTYPE_CODE[torch.float16]);
        the one-call path only."""
        B, H, T, S, dim, mh, mh_valid = self.shape
        if dropout[0] > 0 and (self.n_parts != self.planned_parts or not self.operand_images or local_context != self.local_context):
            raise NotImplementedError('dropout needs the one-call path of the plan (its own part count and band)')
        if io_code and (self.n_parts != self.planned_parts or not self.operand_images or local_context != self.local_context
                        or self.flags):
            raise NotImplementedError('float16 tensors are read as they are on the one-call path of a plan with operand images')
        if self.n_parts != self.planned_parts or not self.operand_images or local_context != self.local_context:
            # a part count or band the library would not choose itself: the two-call path takes them as arguments
            with torch.cuda.device(self.device):
                stream = _lib.stream_ptr(self.device)
                self.run_keys(q, k, v, proj, lens, t, stream)
                self.run_queries(q, k, v, proj, lens, local_context, t, out, log_norm, stream)
            return
        ws = self._workspace()
        with torch.cuda.device(self.device):
            _lib.call('flyhip_sblocal_forward', q.data_ptr(), k.data_ptr(), v.data_ptr(), proj.data_ptr(), _lib.ptr(lens),
                      out.data_ptr(), log_norm.data_ptr(), ws.data_ptr(), ws.numel(),
                      B, H, T, S, dim, dim, mh, mh_valid, local_context,
                      q.stride(0), q.stride(2), q.stride(1), k.stride(0), k.stride(2), k.stride(1),
                      v.stride(0), v.stride(2), v.stride(1), out.stride(0), out.stride(2), out.stride(1),
                      t, self.code | (io_code << 8), self.flags, float(dropout[0]), int(dropout[1]),
                      _lib.stream_ptr(self.device))


class ScratchCache:
    """What a caller keeps between forwards so that a repeated call allocates nothing but its results: the plans
    (device scratch) of the most recently used problem shapes and the padded projection.

    At most ``max_plans`` plans are kept, least recently used dropped first (a plan holds the scratch of its shape:
    roughly 200 MB at batch 64, L = 3136); callers with ever-changing sequence lengths therefore do not grow device
    memory without bound.  The cache is per process and per object: copies and pickles of its owner start empty."""

    def __init__(self, max_plans=4):
        self.max_plans = max_plans
        self.plans = {}                  # insertion-ordered: oldest use first
        self._proj_src = None            # weak reference to the caller's projection tensor the padded copy was made from
        self._proj_stamp = None
        self._proj = None

    def plan(self, key, make):
        got = self.plans.pop(key, None)
        if got is None:
            got = make()
            while len(self.plans) >= self.max_plans:
                self.plans.pop(next(iter(self.plans)))
        self.plans[key] = got            # (re-)inserted as the most recent
        return got

    def padded_projection(self, projection_matrix, mh, dim):
        """The padded float32 copy of `projection_matrix`, remade when the caller's tensor is another object than the
        one the copy was made from (same address and version are not enough: a replaced buffer often gets both)
        or has been written to since."""
        src = None if self._proj_src is None else self._proj_src()
        stamp = (projection_matrix._version, mh, dim, projection_matrix.device)
        if src is projection_matrix and stamp == self._proj_stamp:
            return self._proj
        self._proj = _pad_projection(projection_matrix, mh, dim)
        self._proj_src, self._proj_stamp = weakref.ref(projection_matrix), stamp
        return self._proj

    def clear(self):
        self.plans.clear()
        self._proj_src = self._proj_stamp = self._proj = None

    def __len__(self):
        return len(self.plans)

    def __deepcopy__(self, memo):
        return ScratchCache(self.max_plans)

    def __reduce__(self):
        return (ScratchCache, (self.max_plans,))


def _pad_projection(projection_matrix, mh, dim):
    mh_valid, E = projection_matrix.shape
    proj = torch.zeros(mh, dim, dtype=torch.float32, device=projection_matrix.device)
    proj[:mh_valid, :E] = projection_matrix.to(torch.float32)
    return proj


def _padded_projection(projection_matrix, mh, dim, cache):
    """The projection as the kernels want it: float32, (mh, dim), zero rows / columns as padding.  The caller's
    tensor itself when it already has that form; otherwise a padded copy, kept in `cache` (a ScratchCache) until the
    caller's tensor is replaced or written to."""
    if (tuple(projection_matrix.shape) == (mh, dim) and projection_matrix.dtype == torch.float32
            and projection_matrix.is_contiguous()):
        return projection_matrix
    if cache is None:
        return _pad_projection(projection_matrix, mh, dim)
    return cache.padded_projection(projection_matrix, mh, dim)


def sblocal_forward(query, key, value, projection_matrix, local_context, softmax_temp=None,
                    key_lengths=None, cache=None, exact_fp32=False, dropout_p=0.0, dropout_seed=0):
    """Scatterbrain-local attention forward on the GPU.

    query (B,T,H,E), key (B,S,H,E), value (B,S,H,D) float32 or bfloat16 CUDA tensors (float16 with head dims up to 64 and up
    to 128 features: float32 arithmetic on the values as they are, no widened copies);
    projection_matrix (m/2, E); key_lengths (B,) int64 or None.  Computes what
    sblocal_attention.py:73-122 computes for causal=False, attn_mask=None, eps=0, no dropout.
    Returns (out (B,T,H,D) in the input dtype, log_normalization (B,H,T,1) float32).

    cache: an optional ScratchCache the caller keeps between calls (SBLocalAttention keeps one per module).  It
    holds the plans -- the device scratch -- of the last few problem shapes and the padded projection, so that a
    repeated call allocates nothing but its two results.  Calls that share a cache share scratch: one at a time.

    exact_fp32: float32 inputs only.  False (default): products on the bf16 matrix pipe from operands split into bf16
    pieces with fp32 accumulation (V rounded to 16, the features to 17 significant bits; about 5e-6 of the float64
    result at the benchmark configuration).  True: every product on the fp32 matrix pipe (about 1e-6; 1.6 times the time).

    dropout_p, dropout_seed: dropout of the exact band weights exp(QK - log_normalization) (sblocal_attention.py:116-119:
    the normaliser and the low-rank part see none) inside the band kernel.  No mask is stored: a weight is kept
    according to a hash of (seed, batch, head, query, key), which the backward kernels evaluate again, and kept
    weights are scaled by 1 / (1 - p).  float32 inputs with head dims <= 64 and <= 128 features.
    """
    _lib.require_gpu(query, key, value, projection_matrix, key_lengths)
    if query.dtype not in (torch.float32, torch.bfloat16, torch.float16):
        raise NotImplementedError(f'SBLocal kernels support float32, bfloat16 and float16, got {query.dtype}')
    if key.dtype != query.dtype or value.dtype != query.dtype:
        raise ValueError('query, key and value must share a dtype')
    B, T, H, E = query.shape
    Bk, S, Hk, Ek = key.shape
    Bv, Sv, Hv, D = value.shape
    if (Bk, Hk, Ek) != (B, H, E) or (Bv, Sv, Hv) != (B, S, H):
        raise ValueError(f'inconsistent shapes q{tuple(query.shape)} k{tuple(key.shape)} v{tuple(value.shape)}')
    if projection_matrix.dim() != 2 or projection_matrix.shape[1] != E:
        raise ValueError(f'projection_matrix must be (m/2, {E}), got {tuple(projection_matrix.shape)}')
    if local_context < 1:
        raise ValueError('local_context must be >= 1')
    t = softmax_temp or 1 / math.sqrt(E)          # sblocal_attention.py:59: 0 / None mean "unset"

    dim = _round_up_choice(max(E, D), _HEAD_DIMS, 'head dimension')
    mh_valid = projection_matrix.shape[0]
    mh = _round_up_choice(mh_valid, _FEATURE_ROWS, 'number of projection rows')
    m = 2 * mh

    def prep(x):
        if x.shape[-1] != dim:
            x = F.pad(x, (0, dim - x.shape[-1]))      # zero columns change neither dots nor norms
        return x if _vector_ready(x) else x.contiguous()
    q, k, v = prep(query), prep(key), prep(value)
    proj = _padded_projection(projection_matrix, mh, dim, cache)
    lens = None
    if key_lengths is not None:
        lens = key_lengths.to(device=query.device, dtype=torch.int64).contiguous()
        if lens.shape != (B,):
            raise ValueError(f'key_lengths must have shape ({B},)')

    exact_fp32 = bool(exact_fp32) and query.dtype == torch.float32
    # float16 tensors: the float32 plan on operand images, whose kernels widen what they load and round what they store
    io_code, plan_dtype = 0, query.dtype
    if query.dtype == torch.float16:
        if dim > 64 or m > 128:
            raise NotImplementedError('float16 tensors are read by the kernels on operand images: head dims up to 64, up '
                                      f'to 128 features (got {max(E, D)}, {2 * mh_valid}); widen them to float32')
        io_code, plan_dtype = _lib.DTYPE_CODE[torch.float16], torch.float32
    plan_key = (B, H, T, S, dim, mh, mh_valid, plan_dtype, query.device, local_context, exact_fp32)

    def make_plan():
        return SBLocalPlan(B, H, T, S, dim, mh, mh_valid, plan_dtype, query.device, local_context,
                           exact_fp32=exact_fp32)
    plan = make_plan() if cache is None else cache.plan(plan_key, make_plan)
    out = torch.empty(B, T, H, dim, dtype=query.dtype, device=query.device)
    log_norm = torch.empty(B, H, T, dtype=torch.float32, device=query.device)
    if dropout_p > 0 and (plan_dtype != torch.float32 or exact_fp32 or dim > 64 or m > 128):
        raise NotImplementedError('attention dropout is implemented in the band kernel on bf16 pieces: float32 inputs, '
                                  f'head dims <= 64, <= 128 features (got {query.dtype}, {max(E, D)}, {2 * mh_valid})')
    plan.run(q, k, v, proj, lens, local_context, t, out, log_norm, dropout=(float(dropout_p), int(dropout_seed)),
             io_code=io_code)
    return out[..., :D], log_norm.unsqueeze(-1)


def sbblocksparse_forward_supported(block, dtype, E, D, n_projection_rows, layout_heads, H):
    """Whether sbblocksparse_forward applies: blocks of 16 x 16 or 32 x 32, one layout per attention head, float32 --
    or bfloat16 / float16 where the kernels on operand images run (head dims up to 64, up to 64 projection rows)."""
    fits = block in (16, 32) and max(E, D) <= _HEAD_DIMS[-1] and n_projection_rows <= _FEATURE_ROWS[-1] and layout_heads == H
    if dtype in (torch.bfloat16, torch.float16):
        return fits and max(E, D) <= 64 and n_projection_rows <= 64
    return fits and dtype == torch.float32


def sbblocksparse_forward(query, key, value, projection_matrix, tables, softmax_temp=None, cache=None,
                          dropout_p=0.0, dropout_seed=0):
    """Scatterbrain attention on a block-sparse support (sbblocksparse_attention.py:109-213 for
    need_weights=False; dropout_p, dropout_seed: the dropout of the exact weights of :200, by the hash mask of
    sblocal_forward) on the fused kernels: exact softmax weights on the nonzero blocks (16 x 16 or
    32 x 32), the Performer estimate everywhere else, one normaliser.  query (B,T,H,E), key (B,S,H,E), value
    (B,S,H,D) float32 GPU tensors (bfloat16 / float16 with head dims up to 64 and up to 64 projection rows: read and
    written as they are by the kernels on operand images, the arithmetic is the float32 path's), T and S multiples of the block size; tables = blocksparse_utils.tile_mask_table(layout,
    block) as int32 tensors on the device, optionally followed by union_order(tables[0], H), or the six entries of
    sbblocksparse_attention.fused_tables (start order with the long lists marked, those lists, their parts).
    cache: an optional ScratchCache kept by the caller (plan and padded projection, as for sblocal_forward).
    Returns (out (B,T,H,D), log_normalization (B,H,T,1))."""
    _lib.require_gpu(query, key, value, projection_matrix)
    B, T, H, E = query.shape
    S, D = key.shape[1], value.shape[3]
    if T % 16 or S % 16:
        raise ValueError(f'sequence lengths {T}, {S} must be multiples of the block size (16 or 32)')
    t = softmax_temp or 1 / math.sqrt(E)
    dim = _round_up_choice(max(E, D), _HEAD_DIMS, 'head dimension')
    mh_valid = projection_matrix.shape[0]
    mh = _round_up_choice(mh_valid, _FEATURE_ROWS, 'number of projection rows')

    def prep(x):
        if x.shape[-1] != dim:
            x = F.pad(x, (0, dim - x.shape[-1]))
        return x if _vector_ready(x) else x.contiguous()
    q, k, v = prep(query), prep(key), prep(value)
    proj = _padded_projection(projection_matrix, mh, dim, cache)

    # tile images of the key pass (the band kernel on bf16 pieces) where that kernel exists
    images = dim <= 64 and mh <= 64

    io_code = 0
    if query.dtype != torch.float32:
        if not (images and query.dtype in (torch.bfloat16, torch.float16)
                and key.dtype == query.dtype and value.dtype == query.dtype):
            raise NotImplementedError('sbblocksparse_forward takes float32 tensors, or bfloat16 / float16 ones with head '
                                      f'dims up to 64 and up to 64 projection rows (got {query.dtype}, {dim}, {mh})')
        io_code = _lib.DTYPE_CODE[query.dtype]

    def make_plan():
        return SBLocalPlan(B, H, T, S, dim, mh, mh_valid, torch.float32, query.device, 64, n_parts=1,
                           operand_images=images)
    plan_key = ('block-sparse', B, H, T, S, dim, mh, mh_valid, torch.float32, query.device, images)
    plan = make_plan() if cache is None else cache.plan(plan_key, make_plan)
    out = torch.empty(B, T, H, dim, dtype=query.dtype, device=query.device)
    log_norm = torch.empty(B, H, T, dtype=torch.float32, device=query.device)
    if not 0.0 <= dropout_p < 1.0:
        raise ValueError(f'dropout probability {dropout_p} not in [0, 1)')
    plan.run_block_sparse(q, k, v, proj, t, tables, out, log_norm, dropout=(float(dropout_p), int(dropout_seed)),
                          io_code=io_code)
    return out[..., :D], log_norm.unsqueeze(-1)


class _SBLocalFn(torch.autograd.Function):
    """sblocal_forward with gradients for query, key and value (the projection is a buffer).  The
    forward is the fused kernel path; the backward is sblocal_backward.sblocal_backward."""

    @staticmethod
    def forward(ctx, query, key, value, projection_matrix, local_context, softmax_temp, key_lengths, cache=None,
                exact_fp32=False, dropout_p=0.0, dropout_seed=0):
        out, log_norm = sblocal_forward(query, key, value, projection_matrix, local_context,
                                        softmax_temp=softmax_temp, key_lengths=key_lengths, cache=cache,
                                        exact_fp32=exact_fp32, dropout_p=dropout_p, dropout_seed=dropout_seed)
        ctx.save_for_backward(query, key, value, projection_matrix, out, log_norm)
        ctx.args = (local_context, softmax_temp, key_lengths)
        ctx.dropout = (float(dropout_p), int(dropout_seed))
        ctx.mark_non_differentiable(log_norm)
        return out, log_norm

    @staticmethod
    def backward(ctx, grad_out, _grad_log_norm):
        from .sblocal_backward import sblocal_backward
        query, key, value, projection_matrix, out, log_norm = ctx.saved_tensors
        local_context, softmax_temp, key_lengths = ctx.args
        dq, dk, dv = sblocal_backward(query, key, value, projection_matrix, local_context, softmax_temp,
                                      key_lengths, out, log_norm, grad_out, dropout=ctx.dropout)
        return dq, dk, dv, None, None, None, None, None, None, None, None


def sblocal_attention_fn(query, key, value, projection_matrix, local_context, softmax_temp=None,
                         key_lengths=None, cache=None, exact_fp32=False, dropout_p=0.0, dropout_seed=0):
    """sblocal_forward, differentiable with respect to query, key and value."""
    if torch.is_grad_enabled() and any(x.requires_grad for x in (query, key, value)):
        return _SBLocalFn.apply(query, key, value, projection_matrix, local_context, softmax_temp, key_lengths, cache,
                                exact_fp32, dropout_p, dropout_seed)
    return sblocal_forward(query, key, value, projection_matrix, local_context, softmax_temp=softmax_temp,
                           key_lengths=key_lengths, cache=cache, exact_fp32=exact_fp32, dropout_p=dropout_p,
                           dropout_seed=dropout_seed)


class SBLocalAttention(nn.Module):
    """Local (banded) softmax attention plus a Performer low-rank estimate of everything outside
    the band, under one normaliser.  Query i attends exactly to keys j with
    -(local_context // 2) <= j - i < (local_context + 1) // 2 and through random features to the rest.

    Same constructor and forward signature as the reference class (sblocal_attention.py:29-44).
    The GPU path covers what the reference itself exercises: non-causal, an attn_mask that hides no pair inside the
    band (one that does fails the reference's own assertion, and so it does here), optional
    length-style key_padding_mask, softmax_eps = 0; attention dropout in training mode for float32 inputs with head
    dims <= 64 and <= 128 features (inside the band kernel, see sblocal_forward).  ``need_weights`` /
    ``return_attn_unnormalized`` (:124-136) give the dense matrix for small problems, formed with library products around
    the fused kernels' ``log_normalization``; ``out`` always comes from the kernels.  Any other request raises
    NotImplementedError -- there is no slower fallback inside this module.
    """

    def __init__(self, local_context, dim_heads, nb_features=None, ortho_scaling=0,
                 causal=False, softmax_temp=None, attention_dropout=0.0, softmax_eps=0.0,
                 device=None, dtype=None):
        super().__init__()
        self.feature_map = SBPerformerFeatures(dim_heads, nb_features, ortho_scaling=ortho_scaling,
                                               softmax_temp=softmax_temp, eps=softmax_eps,
                                               device=device, dtype=dtype)
        self.local_context = local_context
        self.causal = causal
        self.softmax_temp = softmax_temp
        self.dropout = nn.Dropout(attention_dropout)
        self.softmax_eps = softmax_eps
        # device scratch of the last few problem shapes and the padded projection, kept between calls (see sblocal_forward)
        self._scratch_cache = ScratchCache()
        # float32 inputs: True selects the fp32 matrix pipe for every product instead of bf16 pieces (see sblocal_forward)
        self.exact_fp32 = False
        # need_weights builds the dense (B,H,T,S) matrix with library products: an inspection aid, not a fast path
        self.max_weight_elements = 1 << 26

    def forward(self, query, key, value, attn_mask=None, key_padding_mask=None, need_weights=False,
                return_attn_unnormalized=False):
        """query (B,T,H,E), key (B,S,H,E), value (B,S,H,D) -> (out (B,T,H,D), None)."""
        if self.causal:
            raise NotImplementedError('causal SBLocalAttention is not implemented (the reference '
                                      'marks it unverified, sblocal_attention.py:61)')
        if attn_mask is not None and not bool(attn_mask.all_ones):
            # The reference adds the mask's -1e24 to the band entries of Q K^T and of Q' K'^T alike (:90-97) and then
            # asserts that the latter are >= 0 (:105): a mask that hides any pair inside the band fails that assertion,
            # and a mask that only hides pairs outside the band changes nothing (the low-rank part never sees it).
            T, S = query.shape[1], key.shape[1]
            hidden = ~attn_mask.bool_matrix
            idx = torch.arange(S, device=hidden.device).view(1, S) - torch.arange(T, device=hidden.device).view(T, 1)
            band = (idx >= -(self.local_context // 2)) & (idx < (self.local_context + 1) // 2)
            if key_padding_mask is not None:
                band = band & (torch.arange(S, device=hidden.device).view(1, S) < int(key_padding_mask.lengths.max()))
            if bool((hidden & band).any()):
                raise AssertionError('attn_mask hides a pair inside the band: the reference adds -1e24 to its feature '
                                     'product and fails its own assertion (sblocal_attention.py:105)')
        if (need_weights or return_attn_unnormalized) and (
                query.shape[0] * query.shape[2] * query.shape[1] * key.shape[1] > self.max_weight_elements):
            raise NotImplementedError('need_weights=True materialises the (B,H,T,S) matrix; supported for inspection '
                                      f'of small problems only (at most {self.max_weight_elements} elements)')
        if self.softmax_eps != 0.0:
            raise NotImplementedError('softmax_eps != 0 is not supported by the fused kernel')
        # attention dropout (:116-119) runs inside the band kernel: a fresh seed per call from the CPU generator
        # (torch.manual_seed makes a run reproducible; no device synchronisation), the mask never exists in memory
        dropout_p, dropout_seed = 0.0, 0
        if self.training and self.dropout.p > 0.0:
            if need_weights or return_attn_unnormalized:
                raise NotImplementedError('need_weights with active attention dropout is not implemented')
            dropout_p = float(self.dropout.p)
            dropout_seed = int(torch.randint(0, 2 ** 62, (1,)).item())
            self.last_dropout_seed = dropout_seed
        lengths = None
        if key_padding_mask is not None and not bool(key_padding_mask.all_ones):
            lengths = key_padding_mask.lengths          # raises ValueError unless a length mask
        self.feature_map.new_feature_map(query.device)
        # float16 inputs (the reference's modules take whatever dtype autocast hands them): the arithmetic is float32
        # either way (exact widening; the feature exponentials do not fit float16's range).  Without gradients the
        # kernels on operand images read them as they are and store the float16 result (head dims up to 64, up to 128
        # features); otherwise they are widened here and the result goes back to float16, the casts being ordinary
        # autograd nodes
        in_dtype = query.dtype
        needs_grad = torch.is_grad_enabled() and any(x.requires_grad for x in (query, key, value))
        as_it_is = (in_dtype == torch.float16 and not needs_grad and not self.exact_fp32
                    and max(query.shape[3], value.shape[3]) <= 64 and self.feature_map.projection_matrix.shape[0] <= 64)
        if in_dtype == torch.float16 and not as_it_is:
            query, key, value = query.float(), key.float(), value.float()
        out, log_norm = sblocal_attention_fn(query, key, value, self.feature_map.projection_matrix,
                                             self.local_context, softmax_temp=self.softmax_temp,
                                             key_lengths=lengths, cache=self._scratch_cache,
                                             exact_fp32=self.exact_fp32, dropout_p=dropout_p, dropout_seed=dropout_seed)
        if in_dtype == torch.float16 and not as_it_is:
            out = out.to(in_dtype)
        self.last_log_normalization = log_norm.detach()
        attn = None
        if need_weights or return_attn_unnormalized:
            attn = self._dense_weights(query.detach(), key.detach(), lengths, log_norm.detach(),
                                       return_attn_unnormalized)
        return out, attn

    def _dense_weights(self, query, key, lengths, log_norm, unnormalized):
        """The (B,H,T,S) attention matrix the output corresponds to (sblocal_attention.py:124-136), for inspection of
        small problems: exact weights exp(t q.k - log_normalization) inside the band, Performer weights
        q'.k' exp(prime_log_scale - log_normalization) outside it, with ``log_normalization`` taken from the fused
        kernels (nothing here feeds back into ``out``).  With ``unnormalized`` the reference's triple
        (attn, attn * exp(log_normalization), attn_prime * exp(prime_log_scale))."""
        B, T, H, E = query.shape
        S = key.shape[1]
        t = self.softmax_temp or 1 / math.sqrt(E)
        q, k = query.permute(0, 2, 1, 3).float(), key.permute(0, 2, 1, 3).float()
        P = self.feature_map.projection_matrix.float()
        q_prime, q_ls = softmax_kernel(q, projection_matrix=P, is_query=True, softmax_temp=t)
        k_prime, k_ls = softmax_kernel(k, projection_matrix=P, is_query=False, softmax_temp=t)
        j = torch.arange(S, device=query.device)
        valid = torch.ones(B, 1, 1, S, dtype=torch.bool, device=query.device) if lengths is None \
            else (j.view(1, 1, 1, S) < lengths.view(B, 1, 1, 1))
        k_prime = k_prime * valid.transpose(-1, -2)                        # :83-85
        prime_log_scale = q_ls + k_ls                                      # (B,H,T,1)
        ln = log_norm.float()                                              # (B,H,T,1)
        attn_prime = q_prime @ k_prime.transpose(-1, -2)
        idx = j.view(1, S) - torch.arange(T, device=query.device).view(T, 1)
        band = ((idx >= -(self.local_context // 2)) & (idx < (self.local_context + 1) // 2)).view(1, 1, T, S) & valid
        exact = torch.exp(t * (q @ k.transpose(-1, -2)) - ln)
        attn = torch.where(band, exact, attn_prime * torch.exp(prime_log_scale - ln))
        if not unnormalized:
            return attn
        return attn, attn * torch.exp(ln), attn_prime * torch.exp(prime_log_scale)
