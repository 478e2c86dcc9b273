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
touch.  Everything is ordinary tensor algebra (library GEMMs on whatever device the tensors
live on); the clamp of the low-rank normaliser (sblocal_attention.py:111) is taken as inactive.
"""
import math

import torch

from .feature_maps_sb import softmax_kernel


def sblocal_backward(query, key, value, projection_matrix, local_context, softmax_temp, key_lengths,
                     out, log_normalization, grad_out, chunk=256):
    """query (B,T,H,E), key (B,S,H,E), value (B,S,H,D), out / grad_out (B,T,H,D),
    log_normalization (B,H,T,1) as returned by the forward; key_lengths (B,) or None.
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

    phiq, lsq = softmax_kernel(Q, projection_matrix=P, is_query=True, softmax_temp=t)
    phik, lsk = softmax_kernel(K, projection_matrix=P, is_query=False, softmax_temp=t)
    lens = None
    if key_lengths is not None:
        lens = key_lengths.to(Q.device).repeat_interleave(H).view(B * H, 1, 1)
        phik = phik * (torch.arange(S, device=Q.device).view(1, S, 1) < lens)
    psi = phiq * torch.exp(lsq + lsk - LN)       # Phi(q_i) Phi(k_s) / Z_i = psi_i . phik_s
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

    for i0 in range(0, T, chunk):
        i1 = min(T, i0 + chunk)
        s0, s1 = max(0, i0 - lc_lo), min(S, i1 - 1 + lc_hi)
        if s1 <= s0:
            continue
        qi, gi, psi_i = Q[:, i0:i1], G[:, i0:i1], psi[:, i0:i1]
        ks, vs, pk = K[:, s0:s1], V[:, s0:s1], phik[:, s0:s1]
        rel = torch.arange(s0, s1, device=Q.device).view(1, -1) - torch.arange(i0, i1, device=Q.device).view(-1, 1)
        band = ((rel >= -lc_lo) & (rel < lc_hi)).unsqueeze(0)
        if lens is not None:
            band = band & (torch.arange(s0, s1, device=Q.device).view(1, 1, -1) < lens)
        band = band.to(wdt)
        a_bar = torch.exp(t * (qi @ ks.transpose(1, 2)) - LN[:, i0:i1]) * band
        k_bar = (psi_i @ pk.transpose(1, 2)) * band
        df = (gi @ vs.transpose(1, 2) - c[:, i0:i1]) * band
        dm = a_bar * df
        dQ[:, i0:i1] += t * (dm @ ks)
        dK[:, s0:s1] += t * (dm.transpose(1, 2) @ qi)
        dV[:, s0:s1] += (a_bar - k_bar).transpose(1, 2) @ gi
        uq[:, i0:i1] -= psi_i * (df @ pk)
        uk[:, s0:s1] -= pk * (df.transpose(1, 2) @ psi_i)

    st = math.sqrt(t)
    dQ += st * ((uq[..., :mh] - uq[..., mh:]) @ P) - t * Q * uq.sum(-1, keepdim=True)
    dK += st * ((uk[..., :mh] - uk[..., mh:]) @ P) - t * K * uk.sum(-1, keepdim=True)

    def back(x, like):                           # (B*H, L, C) -> (B,L,H,C)
        return x.reshape(B, H, x.shape[1], x.shape[2]).permute(0, 2, 1, 3).to(like.dtype)
    return back(dQ, query), back(dK, key), back(dV, value)
