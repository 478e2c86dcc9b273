"""Gradients of Scatterbrain-local attention with respect to query, key and value.

The forward (sblocal_attention.py:73-122 of the reference) gives every query i normalised weights
W_is over ALL keys: exp(t q_i.k_s) / Z_i inside the band, Phi(q_i).Phi(k_s) / Z_i outside it, with
Z_i = exp(log_normalization_i); out_i = sum_s W_is v_s.  The reference obtains the gradients from
autograd through its op sequence and the backward kernels of fast_transformers.local_product.
Here they are written out.  With g = d out, c_i = g_i.out_i and Df_is = g_i.v_s - c_i:

  d v_s   = sum_i W_is g_i
  d(t q_i.k_s) = W_is Df_is                               inside the band
  u_ir    = sum_{s outside} Df_is  Phi_r(q_i) Phi_r(k_s) / Z_i   (gradient w.r.t. log Phi_r(q_i))
  uk_sr   = sum_{i: s outside} the same summand                  (gradient w.r.t. log Phi_r(k_s))
  log Phi_r(x) = +-sqrt(t) p_r.x - t |x|^2 / 2 + const   =>   d x = sqrt(t) P^T (u+ - u-) - t x sum_r u_r

Sums over "outside the band" are taken as (sum over all keys) - (sum over the band): the first is a
product with the global reductions K'^T V, sum K' (queries) or Q'^T g, Q'^T c (keys), the second
a band-limited product evaluated for chunks of queries against the slice of keys their bands
touch -- all chunks at once as batched products over overlapping windows of the keys (BandWindows).
Everything is ordinary tensor algebra (library GEMMs on whatever device the tensors live on); the
clamp of the low-rank normaliser (sblocal_attention.py:111) is taken as inactive.
"""
import math

import torch



class BandWindows:
    """Index bookkeeping for band-limited products taken for all chunks of queries at once.

    Queries are cut into n chunks of C (the last one zero-padded); chunk j meets the window of W keys
    starting at key j*C - lc_lo, W = the multiple of C that covers C + local_context - 1.  Query a of a
    chunk and key b of its window are i = jC + a and s = jC - lc_lo + b, so s - i = b - a - lc_lo:
    the band -lc_lo <= s - i < lc_hi is the pattern 0 <= b - a < local_context for every chunk; on
    top of it keys must exist (0 <= s < S) and lie below the key length."""

    def __init__(self, T, S, local_context, chunk, device, lens=None, max_elements=1 << 27):
        self.T, self.S, self.C = T, S, chunk
        self.lc_lo = local_context // 2
        self.n = -(-T // chunk)
        self.P = -(-(chunk + local_context - 1) // chunk)        # chunk-sized pieces per window
        self.W = self.P * chunk
        self.device, self.lens, self.max_elements = device, lens, max_elements
        a = torch.arange(chunk, device=device).view(-1, 1)
        b = torch.arange(self.W, device=device).view(1, -1)
        self.pattern = ((b - a >= 0) & (b - a < local_context)).view(1, 1, chunk, self.W)

    def chunks(self, x):
        """(BH, T, F) -> (BH, n, C, F), zero rows after T."""
        pad = self.n * self.C - self.T
        if pad:
            x = torch.nn.functional.pad(x, (0, 0, 0, pad))
        return x.reshape(x.shape[0], self.n, self.C, x.shape[2])

    def unchunk(self, x):
        return x.reshape(x.shape[0], self.n * self.C, x.shape[3])[:, :self.T]

    def windows(self, x):
        """(BH, S, F) -> view (BH, n, W, F) of the zero-padded keys (windows overlap)."""
        total = (self.n - 1) * self.C + self.W
        xp = torch.nn.functional.pad(x, (0, 0, self.lc_lo, max(0, total - self.lc_lo - self.S)))[:, :total]
        return xp.unfold(1, self.W, self.C).transpose(2, 3)

    def groups(self, batch):
        """Ranges of chunks whose (batch, g, C, W) intermediates stay below max_elements."""
        g = max(1, self.max_elements // (batch * self.C * self.W))
        return [(j0, min(self.n, j0 + g)) for j0 in range(0, self.n, g)]

    def mask(self, j0, j1):
        """(1 or BH, g, C, W) bool: inside the band, key exists and lies below the key length."""
        s = (torch.arange(j0, j1, device=self.device) * self.C - self.lc_lo).view(1, -1, 1, 1) \
            + torch.arange(self.W, device=self.device).view(1, 1, 1, -1)
        ok = (s >= 0) & (s < self.S)
        if self.lens is not None:
            ok = ok & (s < self.lens.view(-1, 1, 1, 1))
        return self.pattern & ok

    def key_accumulator(self, batch, F, dtype):
        """Zeroed (batch, n + P - 1, C, F): the zero-padded key axis cut into chunk-sized pieces."""
        return torch.zeros(batch, self.n + self.P - 1, self.C, F, dtype=dtype, device=self.device)

    def add_windows(self, buf, j0, win):
        """Overlap-add windows j0.. (BH, g, W, F): piece p of window j lands on key chunk j + p."""
        BH, g, F = win.shape[0], win.shape[1], win.shape[3]
        wv = win.reshape(BH, g, self.P, self.C, F)
        for p in range(self.P):
            buf[:, j0 + p:j0 + p + g] += wv[:, :, p]

    def fold(self, buf):
        """Accumulated windows -> (BH, S, F)."""
        F = buf.shape[3]
        flat = buf.reshape(buf.shape[0], -1, F)                 # row r is key r - lc_lo
        out = flat.new_zeros(buf.shape[0], self.S, F)
        hi = min(flat.shape[1], self.lc_lo + self.S)
        out[:, :hi - self.lc_lo] = flat[:, self.lc_lo:hi]
        return out


_BAND_KERNEL_FEATURES = {32: (32, 64), 64: (32, 64, 128)}       # head dim -> feature counts the band kernels are built for


def _band_kernel_dims(E, D, M):
    """(head dim, feature count) of the band kernels that fit (zero padding up to them changes no
    product), or None."""
    for dim, feats in _BAND_KERNEL_FEATURES.items():
        if max(E, D) <= dim:
            for m in feats:
                if M <= m:
                    return dim, m
    return None


def _fit(x, width):
    if x.shape[-1] != width:
        x = torch.nn.functional.pad(x, (0, width - x.shape[-1]))
    return x.contiguous()


def _fit_features(x, mk):
    """(.., 2 mh) -> (.., mk) keeping the two halves (exp(+.), exp(-.)) at f and f + mk/2."""
    mh = x.shape[-1] // 2
    if 2 * mh == mk:
        return x.contiguous()
    pad = (0, mk // 2 - mh)
    return torch.cat([torch.nn.functional.pad(x[..., :mh], pad), torch.nn.functional.pad(x[..., mh:], pad)], dim=-1)


_SCRATCH_SIZES = {}


def _scratch_sizes(BH, T, S, dim, mk, local_context):
    """Bytes of the two operand-image buffers and floats of the two scratch buffers of the kernel path, as the
    library states them; kept per problem shape."""
    key = (BH, T, S, dim, mk, local_context)
    got = _SCRATCH_SIZES.get(key)
    if got is None:
        from . import _lib
        lib = _lib.load()
        got = {'qimg': lib.flyhip_sblocal_bwd_image_bytes(BH, T, dim, mk),
               'kimg': lib.flyhip_sblocal_bwd_image_bytes(BH, S, dim, mk),
               'scratch': lib.flyhip_sblocal_bwd_prep_scratch(BH, T, S, dim, mk),
               'parts': lib.flyhip_sblocal_bwd_parts_floats(BH, T, S, dim, mk, local_context)}
        if min(got.values()) < 0:
            raise ValueError(f'the backward kernels reject the problem shape {key}')
        if len(_SCRATCH_SIZES) > 256:
            _SCRATCH_SIZES.clear()
        _SCRATCH_SIZES[key] = got
    return got


def _backward_hip(Q, K, V, G, O, LN, P, lens_b, H, local_context, t, dims, pieces=True, support=None, dropout=(0.0, 0)):
    """d query, d key, d value (BH, rows, width) in five launches: flyhip_sblocal_bwd_prep (scaled features of
    queries and keys, c = g . out, and the per-head sums over all keys / all queries) and the two passes of the
    band kernel (everything per (query, key) pair, the low-rank epilogue, the chain rule through the feature map).
    pieces: the band kernel on the bf16 matrix pipe from operands in two bf16 pieces (flyhip_sblocal_bwd_pieces;
    the preparation pass leaves every 32 rows of either side as one image of such operands), else on the fp32
    matrix pipe from the float arrays (flyhip_sblocal_bwd).  support: instead of a band, a block-sparse support of
    16 x 16 or 32 x 32 blocks -- (tables of the query tiles, tables of the key tiles), each (ptr, inner, mask) of
    blocksparse_utils.tile_mask_table(layout, block) resp. tile_mask_table(layout, block, transposed=True) as int32
    tensors on the device, optionally followed by (skip, heavy, parts) for long lists walked in parts
    (sbblocksparse_attention.backward_tables; flyhip_sbblocksparse_bwd_pieces; no key lengths)."""
    from . import _lib
    BH, T, E = Q.shape
    S, D = K.shape[1], V.shape[2]
    dim, mk = dims
    q_, k_, v_, g_, o_ = _fit(Q, dim), _fit(K, dim), _fit(V, dim), _fit(G, dim), _fit(O, dim)
    mh = P.shape[0]
    proj = P.contiguous() if P.shape == (mk // 2, dim) else _fit(torch.nn.functional.pad(P, (0, 0, 0, mk // 2 - mh)), dim)
    ln_ = LN.reshape(BH, T).contiguous()
    new = Q.new_empty
    sizes = _scratch_sizes(BH, T, S, dim, mk, local_context)
    n_ws = sizes['parts']
    psi_ = phik_ = qimg = kimg = part_ws = None
    if pieces:
        images = torch.empty(sizes['qimg'] + sizes['kimg'], dtype=torch.uint8, device=Q.device)
        qimg, kimg = images[:sizes['qimg']], images[sizes['qimg']:]
    else:
        psi_, phik_ = new(BH, T, mk), new(BH, S, mk)
    # the small operands and the scratch as pieces of one allocation (each a multiple of 64 floats long)
    want = [BH * T, BH * mk * dim, BH * mk, BH * mk * dim, BH * mk, sizes['scratch'], n_ws if pieces else 0]
    offs = [0]
    for n in want:
        offs.append(offs[-1] + (n + 63) // 64 * 64)
    pool = new(offs[-1])
    c_, kv, ksum, qg, qc, scratch, ws = (pool[a:a + n] for a, n in zip(offs, want))
    kv, qg = kv.view(BH, mk, dim), qg.view(BH, mk, dim)
    if pieces and n_ws > 0:
        part_ws = ws
    dq, dk, dv = new(BH, T, dim), new(BH, S, dim), new(BH, S, dim)
    with torch.cuda.device(Q.device):
        st = _lib.stream_ptr(Q.device)
        _lib.call('flyhip_sblocal_bwd_prep', q_.data_ptr(), k_.data_ptr(), v_.data_ptr(), g_.data_ptr(), o_.data_ptr(),
                  ln_.data_ptr(), proj.data_ptr(), _lib.ptr(lens_b), _lib.ptr(psi_), _lib.ptr(phik_), c_.data_ptr(),
                  kv.data_ptr(), ksum.data_ptr(), qg.data_ptr(), qc.data_ptr(), _lib.ptr(qimg), _lib.ptr(kimg),
                  scratch.data_ptr(), scratch.numel(), BH, H, T, S, dim, mk, mh, float(t), st)
        if support is not None:
            passes = ((qimg, kimg, q_, kv, ksum, dq, None), (kimg, qimg, k_, qg, qc, dk, dv))
            for key_major, (tabs, (oimg, iimg, x1, gmat, gvec, d1, d3)) in enumerate(zip(support, passes)):
                tl_ptr, tl_inner, tl_blk = tabs[:3]
                skip = heavy = hws = None
                n_heavy, parts, n_hws = 0, 1, 0
                if len(tabs) > 3 and tabs[4].numel() > 0:      # long lists: walked in parts, finished by a second launch
                    skip, heavy, parts = tabs[3], tabs[4], int(tabs[5])
                    n_heavy = heavy.numel()
                    n_hws = _lib.load().flyhip_sbblocksparse_bwd_parts_floats(BH // H, n_heavy, parts, dim, mk, key_major)
                    hws = new(n_hws)
                _lib.call('flyhip_sbblocksparse_bwd_pieces', oimg.data_ptr(), iimg.data_ptr(), x1.data_ptr(), ln_.data_ptr(),
                          c_.data_ptr(), gmat.data_ptr(), gvec.data_ptr(), proj.data_ptr(), d1.data_ptr(), _lib.ptr(d3),
                          tl_ptr.data_ptr(), _lib.table_ptr(tl_inner), _lib.table_ptr(tl_blk), _lib.ptr(skip), _lib.ptr(heavy),
                          n_heavy, parts, _lib.ptr(hws), n_hws, BH, H, T, S, dim, mk, float(t), key_major,
                          float(dropout[0]), int(dropout[1]), st)
        elif pieces:
            _lib.call('flyhip_sblocal_bwd_pieces', qimg.data_ptr(), kimg.data_ptr(), q_.data_ptr(),
                      ln_.data_ptr(), c_.data_ptr(), _lib.ptr(lens_b), kv.data_ptr(), ksum.data_ptr(), proj.data_ptr(),
                      dq.data_ptr(), None, _lib.ptr(part_ws), n_ws, BH, H, T, S, dim, mk, local_context, float(t), 0,
                      float(dropout[0]), int(dropout[1]), st)
            _lib.call('flyhip_sblocal_bwd_pieces', kimg.data_ptr(), qimg.data_ptr(), k_.data_ptr(),
                      ln_.data_ptr(), c_.data_ptr(), _lib.ptr(lens_b), qg.data_ptr(), qc.data_ptr(), proj.data_ptr(),
                      dk.data_ptr(), dv.data_ptr(), _lib.ptr(part_ws), n_ws, BH, H, T, S, dim, mk, local_context, float(t), 1,
                      float(dropout[0]), int(dropout[1]), st)
        else:
            _lib.call('flyhip_sblocal_bwd', q_.data_ptr(), psi_.data_ptr(), g_.data_ptr(), k_.data_ptr(), phik_.data_ptr(),
                      v_.data_ptr(), ln_.data_ptr(), c_.data_ptr(), _lib.ptr(lens_b), kv.data_ptr(), ksum.data_ptr(),
                      proj.data_ptr(), dq.data_ptr(), None, BH, H, T, S, dim, mk, local_context, float(t), 0, st)
            _lib.call('flyhip_sblocal_bwd', k_.data_ptr(), phik_.data_ptr(), v_.data_ptr(), q_.data_ptr(), psi_.data_ptr(),
                      g_.data_ptr(), ln_.data_ptr(), c_.data_ptr(), _lib.ptr(lens_b), qg.data_ptr(), qc.data_ptr(),
                      proj.data_ptr(), dk.data_ptr(), dv.data_ptr(), BH, H, T, S, dim, mk, local_context, float(t), 1, st)
    return dq[..., :E], dk[..., :E], dv[..., :D]


def _band_terms_hip(Q, K, V, G, psi, phik, LN, c, lens_b, H, local_context, t, dims, dropout=(0.0, 0), attn_mask=None):
    """The five band-limited sums on flyhip_sblocal_bwd_band.  Q, G, psi, LN, c: (BH, T, .); K, V, phik:
    (BH, S, .); float32 on the GPU.  Returns (t sum_s dm k, sum_s df phik, t sum_i dm q, sum_i df psi,
    sum_i (a - kb) g) cut back to the callers' widths.  dropout = (p, seed) of a forward that dropped exact
    weights: the kernels form the same mask again from the seed.  attn_mask: the (T, S) float32 additive matrix of
    plain local attention (local_forward), or None."""
    from . import _lib
    BH, T, E = Q.shape
    S, D, M = K.shape[1], V.shape[2], psi.shape[2]
    dim, mk = dims
    q_, k_, v_, g_ = _fit(Q, dim), _fit(K, dim), _fit(V, dim), _fit(G, dim)
    psi_, phik_ = _fit(psi, mk), _fit(phik, mk)
    ln_, c_ = LN.reshape(BH, T).contiguous(), c.reshape(BH, T).contiguous()
    dq, uq = Q.new_empty(BH, T, dim), Q.new_empty(BH, T, mk)
    dk, uk, dv = Q.new_empty(BH, S, dim), Q.new_empty(BH, S, mk), Q.new_empty(BH, S, dim)
    with torch.cuda.device(Q.device):
        st = _lib.stream_ptr(Q.device)
        drop = (float(dropout[0]), int(dropout[1]))
        _lib.call('flyhip_sblocal_bwd_band_masked', q_.data_ptr(), None, g_.data_ptr(), k_.data_ptr(), phik_.data_ptr(),
                  v_.data_ptr(), ln_.data_ptr(), c_.data_ptr(), _lib.ptr(lens_b), _lib.ptr(attn_mask), dq.data_ptr(),
                  uq.data_ptr(), None, BH, H, T, S, dim, mk, local_context, float(t), 0, *drop, st)
        _lib.call('flyhip_sblocal_bwd_band_masked', k_.data_ptr(), phik_.data_ptr(), v_.data_ptr(), q_.data_ptr(),
                  psi_.data_ptr(), g_.data_ptr(), ln_.data_ptr(), c_.data_ptr(), _lib.ptr(lens_b), _lib.ptr(attn_mask),
                  dk.data_ptr(), uk.data_ptr(), dv.data_ptr(), BH, H, T, S, dim, mk, local_context, float(t), 1, *drop, st)
    return dq[..., :E], uq[..., :M], dk[..., :E], uk[..., :M], dv[..., :D]


def _band_terms_torch(Q, K, V, G, psi, phik, LN, c, lens, local_context, t, chunk, max_elements, dQ, dK, dV, uq, uk):
    """The same sums as batched library products, added into dQ, dK, dV, uq, uk (any device, float32 or
    float64)."""
    # band terms, all chunks of queries at once: chunk j (queries jC .. jC+C-1) against the window of
    # keys jC - lc_lo .. jC - lc_lo + W - 1 that its bands touch; inside a window the band is the same
    # (C, W) pattern for every chunk
    BH, T, E = Q.shape
    S, D, mh2, wdt = K.shape[1], V.shape[2], psi.shape[2], Q.dtype
    band = BandWindows(T, S, local_context, chunk, Q.device, lens, max_elements)
    Qc, Gc, Pc, cc, LNc = (band.chunks(x) for x in (Q, G, psi, c, LN))
    acc_k, acc_v, acc_u = (band.key_accumulator(BH, F, wdt) for F in (E, D, mh2))
    dQc, uqc = torch.zeros_like(Qc), torch.zeros_like(Pc)
    Kw, Vw, PKw = band.windows(K), band.windows(V), band.windows(phik)
    for j0, j1 in band.groups(BH):
        sl = slice(j0, j1)
        ks, vs, pk = Kw[:, sl], Vw[:, sl], PKw[:, sl]               # (BH, g, W, .)
        valid = band.mask(j0, j1).to(wdt)
        a_bar = torch.exp(t * (Qc[:, sl] @ ks.transpose(2, 3)) - LNc[:, sl]) * valid
        k_bar = (Pc[:, sl] @ pk.transpose(2, 3)) * valid
        df = (Gc[:, sl] @ vs.transpose(2, 3) - cc[:, sl]) * valid
        dm = a_bar * df
        dQc[:, sl] = t * (dm @ ks)
        uqc[:, sl] = df @ pk
        band.add_windows(acc_k, j0, t * (dm.transpose(2, 3) @ Qc[:, sl]))
        band.add_windows(acc_v, j0, (a_bar - k_bar).transpose(2, 3) @ Gc[:, sl])
        band.add_windows(acc_u, j0, df.transpose(2, 3) @ Pc[:, sl])
    dQ += band.unchunk(dQc)
    uq -= psi * band.unchunk(uqc)
    dK += band.fold(acc_k)
    dV += band.fold(acc_v)
    uk -= phik * band.fold(acc_u)


def _scaled_features(Q, K, P, t, LN, lens):
    """psi (BH,T,m) and phik (BH,S,m) with psi_i . phik_s = Phi(q_i) . Phi(k_s) / Z_i, the low-rank weight
    of the pair (feature_maps_sb.py:51-82 gives Phi_r(x) = exp(+-sqrt(t) p_r.x - t |x|^2 / 2) / sqrt(m),
    the + half first).  One stabiliser kappa per (batch, head), the largest log-feature of a valid key,
    is taken out of the keys and put into the queries together with -log Z; keys at or past the key
    length get zero features."""
    mh = P.shape[0]
    Pt = (math.sqrt(t) * P).t()
    dq, dk = Q @ Pt, K @ Pt                                              # (BH, rows, mh)
    off = math.log(2 * mh) / 2
    bk = K.square().sum(-1, keepdim=True).mul_(-t / 2).sub_(off)        # (BH, S, 1): log-feature = +-dk + bk
    if lens is not None:
        bk = bk.masked_fill(torch.arange(K.shape[1], device=K.device).view(1, -1, 1) >= lens, -math.inf)
    kappa = (dk.abs().amax(-1, keepdim=True) + bk).amax(1, keepdim=True).nan_to_num_(neginf=0.0)
    bk = bk - kappa
    bq = kappa - LN - Q.square().sum(-1, keepdim=True).mul_(t / 2) - off
    psi, phik = Q.new_empty(*dq.shape[:2], 2 * mh), K.new_empty(*dk.shape[:2], 2 * mh)
    torch.exp(dq + bq, out=psi[..., :mh])
    torch.exp(bq - dq, out=psi[..., mh:])
    torch.exp(dk + bk, out=phik[..., :mh])
    torch.exp(bk - dk, out=phik[..., mh:])
    return psi, phik


def sblocal_backward(query, key, value, projection_matrix, local_context, softmax_temp, key_lengths,
                     out, log_normalization, grad_out, chunk=256, max_elements=1 << 27, band_kernel=None, support=None,
                     dropout=(0.0, 0)):
    """query (B,T,H,E), key (B,S,H,E), value (B,S,H,D), out / grad_out (B,T,H,D),
    log_normalization (B,H,T,1) as returned by the forward; key_lengths (B,) or None.
    max_elements bounds the
    size of the (batch, chunks, chunk, window) intermediates: chunks are taken in groups that stay below it.
    band_kernel: None = the fused kernels where they apply (GPU, head dims <= 64, <= 128 features): the
    feature maps and per-head sums in three launches, then band sums, global low-rank terms and the feature-map
    chain rule in two, on the bf16 matrix pipe from operands in two bf16 pieces; 'fp32' = the same five launches
    with the band kernel on the fp32 matrix pipe; 'sums' = only the band sums on the kernels, the rest as tensor
    algebra; False = batched library products; True = the kernels or NotImplementedError.
    support: the exact part lives on a block-sparse support of 16 x 16 or 32 x 32 blocks instead of a band (Scatterbrain
    attention on a block-sparse support, sbblocksparse_attention.py:161-212): see _backward_hip; kernels only, no key
    lengths, local_context is ignored.
    dropout: (probability, seed) the forward was called with; the band kernels on bf16 pieces form the forward's mask
    again from the seed (other paths: NotImplementedError when the probability is not zero).
    Returns (d query, d key, d value) in the dtypes of the inputs."""
    B, T, H, E = query.shape
    S, D = key.shape[1], value.shape[3]
    t = softmax_temp or 1 / math.sqrt(E)
    lc_lo, lc_hi = local_context // 2, (local_context + 1) // 2
    wdt = torch.float64 if query.dtype == torch.float64 else torch.float32

    def bh(x):                                   # (B,L,H,C) -> (B*H, L, C)
        return x.permute(0, 2, 1, 3).reshape(B * H, x.shape[1], x.shape[3]).to(wdt)
    Q, K, V, G, O = bh(query), bh(key), bh(value), bh(grad_out), bh(out)
    LN = log_normalization.reshape(B * H, T, 1).to(wdt)
    P = projection_matrix.to(wdt)
    mh = P.shape[0]

    lens = None
    if key_lengths is not None:
        lens = key_lengths.to(Q.device).repeat_interleave(H).view(B * H, 1, 1)
    dims = _band_kernel_dims(E, D, 2 * mh) if band_kernel is not False else None
    if band_kernel and dims is None:
        raise NotImplementedError(f'no band kernel for head dims ({E}, {D}) with {2 * mh} features')
    on_kernels = dims is not None and Q.is_cuda and wdt == torch.float32
    if not Q.is_cuda and wdt != torch.float64:
        # host tensors are accepted for one purpose: checking the written-out gradient formulas in float64 against autograd
        raise NotImplementedError('sblocal_backward runs on the GPU; host tensors only in float64 (the check of the formulas)')
    lens_b = None if key_lengths is None else key_lengths.to(device=Q.device, dtype=torch.int64).contiguous()
    if dropout[0] > 0 and (not on_kernels or band_kernel in ('sums', 'fp32')):
        raise NotImplementedError('the backward under attention dropout runs on the band kernels on bf16 pieces only '
                                  f'(GPU, head dims <= 64, <= 128 features; got ({E}, {D}), {2 * mh})')
    if support is not None:
        if not on_kernels or key_lengths is not None or T % 16 or S % 16:
            raise NotImplementedError('the backward on a block-sparse support needs the GPU kernels (float32 or bfloat16 '
                                      f'inputs, head dims <= 64, <= 128 features; got ({E}, {D}), {2 * mh}), sequence '
                                      'lengths that are multiples of 16 and no key lengths')
        dQ, dK, dV = _backward_hip(Q, K, V, G, O, LN, P, None, H, 1, t, dims, support=support, dropout=dropout)
    elif on_kernels and band_kernel != 'sums':
        # features, per-head sums and the two passes of the fused kernel
        dQ, dK, dV = _backward_hip(Q, K, V, G, O, LN, P, lens_b, H, local_context, t, dims,
                                   pieces=band_kernel != 'fp32', dropout=dropout)
    else:
        psi, phik = _scaled_features(Q, K, P, t, LN, lens)
        c = (G * O).sum(-1, keepdim=True)
        kv = phik.transpose(1, 2) @ V                # (BH, m, D)   sum_s phik_s v_s^T
        ksum = phik.sum(1)                           # (BH, m)
        qg = psi.transpose(1, 2) @ G                 # (BH, m, D)   sum_i psi_i g_i^T
        qc = (psi * c).sum(1)                        # (BH, m)
        uq = psi * (G @ kv.transpose(1, 2) - c * ksum.unsqueeze(1))
        uk = phik * (V @ qg.transpose(1, 2) - qc.unsqueeze(1))
        dV = phik @ qg
        dQ = torch.zeros_like(Q)
        dK = torch.zeros_like(K)
        if on_kernels:
            # only the band-limited sums on the kernels
            dQ_b, uq_b, dK_b, uk_b, dV_b = _band_terms_hip(Q, K, V, G, psi, phik, LN, c, lens_b, H, local_context, t, dims)
            dQ += dQ_b
            uq -= psi * uq_b
            dK += dK_b
            uk -= phik * uk_b
            dV += dV_b
        else:
            _band_terms_torch(Q, K, V, G, psi, phik, LN, c, lens, local_context, t, chunk, max_elements,
                              dQ, dK, dV, uq, uk)
        st = math.sqrt(t)
        dQ += st * ((uq[..., :mh] - uq[..., mh:]) @ P) - t * Q * uq.sum(-1, keepdim=True)
        dK += st * ((uk[..., :mh] - uk[..., mh:]) @ P) - t * K * uk.sum(-1, keepdim=True)

    def back(x, like):                           # (B*H, L, C) -> (B,L,H,C)
        # (in the inputs' own memory order: autograd then accumulates the gradient without another copy)
        return x.reshape(B, H, x.shape[1], x.shape[2]).permute(0, 2, 1, 3).to(like.dtype, memory_format=torch.contiguous_format)
    return back(dQ, query), back(dK, key), back(dV, value)
