"""Oracle (test infrastructure) for Scatterbrain-local attention.

Restates, op for op, ``src/models/attention/sblocal_attention.py:43-137`` and what it
calls.  Pinning (see tests/test_oracle_sblocal.py):

* ``gaussian_orthogonal_random_matrix`` -- invariant ``P = diag(row norms) * Q`` with
  ``Q Q^T = I`` per square block.  RNG-stream equality with the reference is not
  claimed (the projection matrix is handed to both sides as data).
* ``softmax_kernel`` -- closed form of the positive random features evaluated by
  brute force in float64.
* ``local_dot_product`` / ``local_weighted_average`` -- brute-force O(T*S) loops on
  tiny inputs; equality with dense attention restricted to the band.
* ``sblocal_attention`` -- ``dense_closed_form`` (an independent float64 evaluation
  of the Scatterbrain estimator written from the mathematics, not from the
  reference's op sequence) plus the invariants of the reference's own test
  (rows sum to one, ``v == 1 -> out == 1``, wide band -> full attention).
"""
import math

import torch


# --------------------------------------------------------------------------------------
# projection matrix -- src/models/attention/projection_utils.py:8-28
# --------------------------------------------------------------------------------------
def gaussian_orthogonal_random_matrix(nrows, ncols, scaling=0, generator=None,
                                      dtype=torch.float32):
    """projection_utils.py:8-28.  Blocks of QR-orthogonalised Gaussians; rows scaled by
    chi-distributed norms (scaling=0) or sqrt(ncols) (scaling=1).  All draws come from one
    CPU generator so that the matrix is reproducible on any box."""
    nblocks = int(math.ceil(nrows / ncols))
    blocks = torch.randn((nblocks, ncols, ncols), generator=generator, dtype=torch.float64)
    q, r = torch.linalg.qr(blocks)
    q = q * torch.diagonal(r, dim1=-2, dim2=-1).sign().unsqueeze(1)   # :15 Haar fix
    q = q.transpose(-1, -2)                                             # :19
    g_ortho = q.reshape(nblocks * ncols, ncols)[:nrows]                 # :20
    if scaling == 0:                                                    # :22-24
        multiplier = torch.randn((nrows, ncols), generator=generator,
                                 dtype=torch.float64).norm(dim=1)
        out = multiplier.unsqueeze(1) * g_ortho
    elif scaling == 1:                                                  # :25-26
        out = math.sqrt(ncols) * g_ortho
    else:
        raise ValueError(f'Invalid scaling {scaling}')
    return out.to(dtype)


# --------------------------------------------------------------------------------------
# feature map -- src/models/attention/feature_maps_sb.py:51-82
# --------------------------------------------------------------------------------------
def softmax_kernel(data, projection_matrix, is_query, softmax_temp=None, eps=0.0):
    """feature_maps_sb.py:51-82 with cosh=True, return_log=False.
    data (..., L, E); projection_matrix (m/2, E).  Returns (features (..., L, m), log_scale)."""
    d = data.shape[-1]
    m = 2 * projection_matrix.shape[0]
    if softmax_temp is None:
        softmax_temp = 1 / math.sqrt(d)
    data_normalizer = math.sqrt(softmax_temp)
    projection_matrix = projection_matrix.to(data.dtype)
    data_dash = torch.einsum('...id,jd->...ij', data, data_normalizer * projection_matrix)
    diag_data = data.square().sum(dim=-1, keepdim=True) / 2 * (data_normalizer ** 2)
    data_dash = torch.cat([data_dash, -data_dash], dim=-1)                       # :66
    if is_query:                                                                  # :67-72
        row_max = torch.amax(data_dash, dim=-1, keepdim=True)
        log_scale = -diag_data + row_max - math.log(m) / 2
        feat = torch.exp(data_dash - row_max) + eps / math.sqrt(m)
    else:                                                                         # :73-78
        z = data_dash - diag_data - math.log(m) / 2
        log_scale = torch.amax(z, dim=(-1, -2), keepdim=True)
        feat = torch.exp(z - log_scale) + eps / math.sqrt(m)
    return feat.to(data.dtype), log_scale


# --------------------------------------------------------------------------------------
# low-rank reductions -- src/models/attention/scatterbrain_utils.py:18-22, 48-52
# --------------------------------------------------------------------------------------
def linear_attention_normalization(q, k):
    """scatterbrain_utils.py:18-20 (non-causal): q' . sum_s k'."""
    return torch.einsum('...nm,...m->...n', q, k.sum(dim=-2))


def linear_attention(q, k, v):
    """scatterbrain_utils.py:48-52 (non-causal, need_weights=False)."""
    k_v = torch.einsum('...nm,...nd->...md', k, v)
    return torch.einsum('...nm,...md->...nd', q, k_v)


# --------------------------------------------------------------------------------------
# fast_transformers.local_product, restated from the call sites
# (sblocal_attention.py:90-105,121; local_attention.py:68-106) and the masks in
# tests/models/attention/test_sblocal_attention.py:77-82.
# --------------------------------------------------------------------------------------
def local_dot_product(Q, K, attn_mask_additive, key_lengths, local_context, chunk=256):
    """out[b,h,i,j] = Q[b,h,i].K[b,h,i - lc//2 + j] + mask[i,s]; -1e24 where the key index
    s = i - lc//2 + j is < 0 or >= key_lengths[b].  Q (B,H,T,E), K (B,H,S,E) -> (B,H,T,lc).
    Evaluated as dense matmuls over query chunks against the keys the chunk can reach."""
    B, H, T, _ = Q.shape
    S = K.shape[2]
    lc = local_context
    out = Q.new_full((B, H, T, lc), -1e24)
    for t0 in range(0, T, chunk):
        t1 = min(T, t0 + chunk)
        s0 = max(0, t0 - lc // 2)
        s1 = min(S, t1 - 1 + (lc + 1) // 2)
        if s1 <= s0:
            continue
        dots = Q[:, :, t0:t1] @ K[:, :, s0:s1].transpose(-1, -2)       # (B,H,tc,sc)
        if attn_mask_additive is not None:
            dots = dots + attn_mask_additive[t0:t1, s0:s1]
        i = torch.arange(t0, t1).view(-1, 1)
        j = torch.arange(lc).view(1, -1)
        s = i - lc // 2 + j                                             # (tc, lc) key index
        inside = (s >= s0) & (s < s1)
        gathered = torch.gather(dots, 3, (s.clamp(s0, s1 - 1) - s0).expand(B, H, -1, -1))
        valid = inside.view(1, 1, t1 - t0, lc) & (s.view(1, 1, t1 - t0, lc)
                                                  < key_lengths.view(B, 1, 1, 1))
        out[:, :, t0:t1] = torch.where(valid, gathered, out[:, :, t0:t1])
    return out


def local_weighted_average(A, V, chunk=256):
    """out[b,h,i] = sum_j A[b,h,i,j] * V[b,h,i - lc//2 + j] over key indices inside [0,S).
    A (B,H,T,lc), V (B,H,S,D) -> (B,H,T,D)."""
    B, H, T, lc = A.shape
    S, D = V.shape[2], V.shape[3]
    out = V.new_zeros((B, H, T, D))
    for t0 in range(0, T, chunk):
        t1 = min(T, t0 + chunk)
        s0 = max(0, t0 - lc // 2)
        s1 = min(S, t1 - 1 + (lc + 1) // 2)
        if s1 <= s0:
            continue
        i = torch.arange(t0, t1).view(-1, 1)
        j = torch.arange(lc).view(1, -1)
        s = i - lc // 2 + j
        inside = (s >= s0) & (s < s1)
        dense = A.new_zeros((B, H, t1 - t0, s1 - s0))
        idx = (s.clamp(s0, s1 - 1) - s0).expand(B, H, -1, -1)
        dense.scatter_add_(3, idx, torch.where(inside.view(1, 1, t1 - t0, lc), A[:, :, t0:t1],
                                               torch.zeros((), dtype=A.dtype)))
        out[:, :, t0:t1] = dense @ V[:, :, s0:s1]
    return out


# --------------------------------------------------------------------------------------
# SBLocalAttention.forward -- src/models/attention/sblocal_attention.py:43-137
# --------------------------------------------------------------------------------------
def _mix32(h):
    """The 32-bit finaliser of MurmurHash3 on int64 tensors holding values below 2^32 (products wrap modulo 2^64, which
    leaves their low 32 bits intact)."""
    m = 0xFFFFFFFF
    h = h ^ (h >> 16)
    h = (h * 0x85EBCA6B) & m
    h = h ^ (h >> 13)
    h = (h * 0xC2B2AE35) & m
    return h ^ (h >> 16)


def dropout_keep(seed, p, B, H, T, S):
    """The dropout multiplier of the HIP kernels, restated on the host so that tests can hand the kernels' own
    mask to the reference algebra: (B,H,T,S) float64, 1 / (1 - p') where the weight of (query i, key s) of (batch b,
    head h) is kept and 0 where it is dropped, p' = floor(p 2^16) 2^-16 the probability actually realised.  A pair of neighbouring keys (2c, 2c + 1) shares the 32-bit hash
    mix(mix(((b H + h) T + i) * 0x9E3779B1 + seed') + c * 0x632BE5AB), key 2c takes its low and key 2c + 1 its high 16
    bits, and a weight is kept iff its half >= floor(p 2^16); seed' is the 64-bit seed folded to 32 bits
    (fly_amd/csrc/common.h: drop_args, drop_row_hash, drop_keep).  This has no counterpart in the reference, whose mask
    comes from torch's generator (sblocal_attention.py:119); the statistics -- independent keeps with probability 1 - p
    (p rounded down to a multiple of 2^-16) -- are what both share."""
    m = 0xFFFFFFFF
    seed32 = (seed & m) ^ (((seed >> 32) * 0x9E3779B1) & m)
    thresh = min(max(int(p * 65536.0), 1), 0xFFFF) if p > 0 else 0
    rows = torch.arange(B * H * T, dtype=torch.int64)
    row_hash = _mix32((rows * 0x9E3779B1 + seed32) & m).view(B, H, T, 1)
    cols = torch.arange(S, dtype=torch.int64).view(1, 1, 1, S)
    h = _mix32((row_hash + (cols >> 1) * 0x632BE5AB) & m)
    half = torch.where((cols & 1) == 1, h >> 16, h & 0xFFFF)
    return (half >= thresh).to(torch.float64) / (1.0 - thresh / 65536.0)


def sblocal_attention(query, key, value, projection_matrix, local_context, softmax_temp=None,
                      key_lengths=None, chunk=256, return_band_lowrank_mass=False, dropout_multiplier=None):
    """sblocal_attention.py:56-122 for causal=False, attn_mask=None, eps=0, dropout off.
    query (B,T,H,E), key (B,S,H,E), value (B,S,H,D); projection_matrix (m/2, E);
    key_lengths (B,) int64 or None.  The reference's ``softmax_temp or 1/sqrt(E)`` (:59)
    treats 0/None as unset.  Returns (out (B,T,H,D), log_normalization (B,H,T,1)); with
    return_band_lowrank_mass also (B,H,T,1): the normalised low-rank weight a query's band carries,
    sum_band q'.k' * prime_scale -- the amount that is subtracted on the band and added back through the
    sums over all keys (a condition number of the estimator: of order one or below when the features
    approximate the exact weights, hundreds when they do not).
    dropout_multiplier: None, or (B,H,T,S) -- the mask of nn.Dropout times 1 / (1 - p) as it falls on the pair (query,
    key); it multiplies exp(QK - log_normalization) and nothing else (:116-119)."""
    B, T, H, E = query.shape
    _, S, _, D = value.shape
    t = softmax_temp or 1 / math.sqrt(E)
    if key_lengths is None:
        key_lengths = torch.full((B,), S, dtype=torch.long)
    q = query.permute(0, 2, 1, 3).contiguous()                                   # :73-75
    k = key.permute(0, 2, 1, 3).contiguous()
    v = value.permute(0, 2, 1, 3).contiguous()

    q_prime, q_ls = softmax_kernel(q, projection_matrix, True, softmax_temp=t)    # :78
    k_prime, k_ls = softmax_kernel(k, projection_matrix, False, softmax_temp=t)   # :79
    prime_log_scale = q_ls + k_ls                                                 # :81
    keep = (torch.arange(S).view(1, S) < key_lengths.view(B, 1))                  # :83-85
    if not bool(keep.all()):
        k_prime = k_prime.masked_fill(~keep.view(B, 1, S, 1), 0.0)
    qk1 = linear_attention_normalization(q_prime, k_prime)                        # :87
    qkv = linear_attention(q_prime, k_prime, v)                                   # :88

    lc = local_context
    QK = t * local_dot_product(q, k, None, key_lengths, lc, chunk)                # :90-93
    dots_prime = local_dot_product(q_prime, k_prime, None, key_lengths, lc, chunk)  # :94-97
    i = torch.arange(T).view(1, 1, T, 1)                                          # :100-105
    j = torch.arange(lc)
    local_idx = i - lc // 2 + j
    valid = (local_idx >= 0) & (local_idx < key_lengths.view(B, 1, 1, 1))
    dots_prime = dots_prime.masked_fill(~valid, 0.0)

    QK_lse = torch.logsumexp(QK, dim=-1, keepdim=True)                            # :109
    dots_prime_sum = dots_prime.sum(dim=-1, keepdim=True)                         # :110
    lr_ln = torch.log((qk1.unsqueeze(-1) - dots_prime_sum).clamp_min(1e-24)) + prime_log_scale
    log_normalization = torch.logaddexp(QK_lse, lr_ln)                            # :113
    prime_scale = torch.exp(prime_log_scale - log_normalization)                  # :115
    exact = torch.exp(QK - log_normalization)
    if dropout_multiplier is not None:                                            # self.dropout(...), :119
        exact = exact * torch.gather(dropout_multiplier.to(exact.dtype), 3, local_idx.clamp(0, S - 1).expand(B, H, T, lc))
    dots = exact - dots_prime * prime_scale                                       # :119
    out = local_weighted_average(dots, v, chunk) + qkv * prime_scale              # :121-122
    if return_band_lowrank_mass:
        return out.permute(0, 2, 1, 3), log_normalization, dots_prime_sum * prime_scale
    return out.permute(0, 2, 1, 3), log_normalization


# --------------------------------------------------------------------------------------
# Independent float64 evaluation of the estimator (pins sblocal_attention)
# --------------------------------------------------------------------------------------
def dense_closed_form(query, key, value, projection_matrix, local_context, softmax_temp=None,
                      key_lengths=None):
    """Scatterbrain-local attention written from the mathematics in float64, O(T*S*m):

        phi(x)_r  = exp(+-w_r . sqrt(t) x - t |x|^2 / 2) / sqrt(m)
        A_ij      = exp(t q_i.k_j)            if j in band(i) and j < len
                    phi(q_i).phi(k_j)         if j outside the band and j < len
                    0                         otherwise
        Z_i = sum_j A_ij ,  out_i = sum_j A_ij v_j / Z_i ,  log_normalization_i = log Z_i

    No stabilisers, no band-packed tensors, no subtraction of the overlap: a different
    route to the same quantity, valid while nothing overflows float64 and the reference's
    1e-24 clamp is inactive.  Returns (out (B,T,H,D), log Z (B,H,T,1), A (B,H,T,S))."""
    B, T, H, E = query.shape
    S = key.shape[1]
    t = softmax_temp or 1 / math.sqrt(E)
    if key_lengths is None:
        key_lengths = torch.full((B,), S, dtype=torch.long)
    q = query.permute(0, 2, 1, 3).double()
    k = key.permute(0, 2, 1, 3).double()
    v = value.permute(0, 2, 1, 3).double()
    W = projection_matrix.double() * math.sqrt(t)
    m = 2 * W.shape[0]

    def phi(x):
        proj = x @ W.t()
        sq = (x * x).sum(-1, keepdim=True) * t / 2
        return torch.exp(torch.cat([proj, -proj], -1) - sq) / math.sqrt(m)

    lowrank = phi(q) @ phi(k).transpose(-1, -2)                    # (B,H,T,S)
    exact = torch.exp(t * (q @ k.transpose(-1, -2)))
    i = torch.arange(T).view(T, 1)
    j = torch.arange(S).view(1, S)
    band = ((j - i) >= -(local_context // 2)) & ((j - i) < (local_context + 1) // 2)
    A = torch.where(band.view(1, 1, T, S), exact, lowrank)
    A = A * (j.view(1, 1, 1, S) < key_lengths.view(B, 1, 1, 1))
    Z = A.sum(-1, keepdim=True)
    out = (A @ v) / Z
    return out.permute(0, 2, 1, 3), torch.log(Z), A


def local_attention(query, key, value, local_context, softmax_temp=None, key_lengths=None, attn_mask_additive=None):
    """LocalAttention.forward without dropout (local_attention.py:50-92; attn_mask_additive = the (T,S)
    additive_matrix_finite of :53-56, default zeros): band-packed
    scores from local_dot_product, softmax over the packed axis, rows without a valid key zeroed when
    a key padding mask is given, local_weighted_average.  query (B,T,H,E) -> out (B,T,H,D)."""
    B, T, H, E = query.shape
    S = key.shape[1]
    t = softmax_temp or 1 / math.sqrt(E)
    q = query.permute(0, 2, 1, 3)
    k = key.permute(0, 2, 1, 3)
    v = value.permute(0, 2, 1, 3)
    lengths = torch.full((B,), S, dtype=torch.long) if key_lengths is None else key_lengths
    add = torch.zeros(T, S, dtype=q.dtype) if attn_mask_additive is None else attn_mask_additive.to(q.dtype)
    QK = local_dot_product(q, k, add, lengths, local_context)                                  # :68-74
    attn = torch.softmax(t * QK, dim=-1)                                                       # :75
    if key_lengths is not None:                                                                # :82-88
        i = torch.arange(T).view(1, 1, T, 1)
        j = torch.arange(local_context)
        idx = i - local_context // 2 + j
        valid = (idx >= 0) & (idx < lengths.view(B, 1, 1, 1))
        attn = attn.masked_fill(~valid, 0.0)
    return local_weighted_average(attn, v).permute(0, 2, 1, 3)                                 # :91
