"""MultiheadAttention wrapper: parameter names of the reference's state dict
(src/models/modules/multihead_attention.py:64-112), the projection packing checked against
torch.nn.MultiheadAttention through a plain softmax attention layer, mask handling of the extra key
positions; on the GPU, the wrapper around SBLocalAttention against the same wrapper around the oracle."""
import math

import pytest
import torch

from fly_amd.masking import FullMask, LengthMask
from fly_amd.multihead_attention import MultiheadAttention


class DenseSoftmaxLayer(torch.nn.Module):
    """(B, T, H, d) attention layer interface over an ordinary softmax; records the masks it is given."""

    def forward(self, q, k, v, attn_mask=None, key_padding_mask=None, need_weights=False):
        self.seen = (attn_mask, key_padding_mask)
        s = torch.einsum('bthd,bshd->bhts', q, k) / math.sqrt(q.shape[-1])
        if key_padding_mask is not None:
            s = s + key_padding_mask.additive_matrix[:, None, None, :]
        if attn_mask is not None:
            s = s + attn_mask.additive_matrix
        p = s.softmax(dim=-1)
        return torch.einsum('bhts,bshd->bthd', p, v), (p if need_weights else None)


def test_state_dict_names():
    base = ['in_proj_weight', 'in_proj_bias', 'in_proj_container.in_proj_weight', 'in_proj_container.in_proj_bias',
            'out_proj.weight', 'out_proj.bias']
    m = MultiheadAttention(64, 4)
    assert list(m.state_dict().keys()) == base
    assert m.in_proj_weight.shape == (192, 64) and m.in_proj_bias.shape == (192,)
    assert m.in_proj_container.in_proj_weight is m.in_proj_weight          # aliases, not copies
    assert float(m.in_proj_bias.detach().abs().max()) == 0.0 and float(m.out_proj.bias.detach().abs().max()) == 0.0
    m = MultiheadAttention(64, 4, shared_qk=True, add_bias_kv=True)
    assert m.in_proj_weight.shape == (128, 64) and m.in_proj_bias.shape == (128,)
    assert set(m.state_dict().keys()) == set(base) | {'bias_k', 'bias_v'}
    assert m.bias_k.shape == (1, 1, 64)
    m = MultiheadAttention(64, 4, kdim=32, vdim=48, bias=False)
    assert set(m.state_dict().keys()) == {'q_proj_weight', 'k_proj_weight', 'v_proj_weight',
                                          'in_proj_container.q_proj_weight', 'in_proj_container.k_proj_weight',
                                          'in_proj_container.v_proj_weight', 'out_proj.weight'}
    assert m.q_proj_weight.shape == (32, 64) and m.v_proj_weight.shape == (48, 64) and m.out_proj.weight.shape == (64, 48)
    m = MultiheadAttention(64, 4, kdim=32, vdim=48, shared_qk=True)
    assert m.k_proj_weight is None and m.in_proj_bias.shape == (32 + 48,)
    # xavier-uniform bound of the packed weight: sqrt(6 / (fan_in + fan_out)) over the PACKED shape
    m = MultiheadAttention(64, 4)
    assert float(m.in_proj_weight.detach().abs().max()) <= math.sqrt(6.0 / (64 + 192)) + 1e-6


@pytest.mark.parametrize('batch_first', [False, True])
@pytest.mark.parametrize('kind', ['self', 'cross', 'all_different'])
@pytest.mark.parametrize('extras', [(False, False), (True, True)])
def test_matches_torch_multihead_attention(batch_first, kind, extras):
    """Same weights in torch.nn.MultiheadAttention: the packed projection order (q | k | v), the head
    split and the output projection have to agree.  torch appends bias_k and the zero position after
    the keys, this wrapper puts them in front; without masks a softmax does not see the order."""
    add_bias_kv, add_zero_attn = extras
    torch.manual_seed(0)
    E, H, B, T, S = 32, 4, 3, 5, 7
    ours = MultiheadAttention(E, H, batch_first=batch_first, add_bias_kv=add_bias_kv, add_zero_attn=add_zero_attn)
    theirs = torch.nn.MultiheadAttention(E, H, batch_first=batch_first, add_bias_kv=add_bias_kv,
                                         add_zero_attn=add_zero_attn)
    with torch.no_grad():
        ours.in_proj_bias.normal_()
        ours.out_proj.bias.normal_()
    sd = {k: v for k, v in ours.state_dict().items() if not k.startswith('in_proj_container.')}
    theirs.load_state_dict(sd)
    shape = (lambda n: (B, n, E)) if batch_first else (lambda n: (n, B, E))
    x = torch.randn(shape(T))
    if kind == 'self':
        q = k = v = x
    elif kind == 'cross':
        q, k = x, torch.randn(shape(S))
        v = k
    else:
        q, k, v = x, torch.randn(shape(S)), torch.randn(shape(S))
    out, w = ours(DenseSoftmaxLayer(), q, k, v)
    ref, _ = theirs(q, k, v, need_weights=False)
    assert w is None and out.shape == ref.shape
    assert torch.allclose(out, ref, rtol=1e-5, atol=1e-6), float((out - ref).abs().max())


def test_shared_qk_and_separate_weights():
    torch.manual_seed(1)
    E, H, B, T = 32, 4, 2, 6
    x = torch.randn(T, B, E)
    layer = DenseSoftmaxLayer()
    m = MultiheadAttention(E, H, shared_qk=True)
    with torch.no_grad():
        m.in_proj_bias.normal_()
    out, _ = m(layer, x, x, x)
    w_qk, w_v = m.in_proj_weight[:E], m.in_proj_weight[E:]
    b_qk, b_v = m.in_proj_bias[:E], m.in_proj_bias[E:]
    qk = torch.nn.functional.linear(x, w_qk, b_qk).transpose(0, 1).reshape(B, T, H, -1)
    vv = torch.nn.functional.linear(x, w_v, b_v).transpose(0, 1).reshape(B, T, H, -1)
    ref = m.out_proj(layer(qk, qk, vv)[0].reshape(B, T, -1)).transpose(0, 1)
    assert torch.allclose(out, ref, rtol=1e-5, atol=1e-6)
    # self-attention (one GEMM) and the same tensors passed as three objects (three GEMMs) agree
    out3, _ = m(layer, x, x.clone(), x.clone())
    assert torch.allclose(out, out3, rtol=1e-5, atol=1e-6)
    m = MultiheadAttention(E, H, kdim=16, vdim=24)
    with torch.no_grad():
        m.in_proj_bias.normal_()
    out, _ = m(layer, x, x, x)
    b_q, b_k, b_v = m.in_proj_bias.split([16, 16, 24])
    qq, kk, vv = (torch.nn.functional.linear(x, w, b).transpose(0, 1).reshape(B, T, H, -1)
                  for w, b in ((m.q_proj_weight, b_q), (m.k_proj_weight, b_k), (m.v_proj_weight, b_v)))
    ref = m.out_proj(layer(qq, kk, vv)[0].reshape(B, T, -1)).transpose(0, 1)
    assert out.shape == (T, B, E) and torch.allclose(out, ref, rtol=1e-5, atol=1e-6)


def test_extra_key_positions_extend_the_masks_on_the_left():
    torch.manual_seed(2)
    E, H, B, T = 16, 2, 2, 4
    m = MultiheadAttention(E, H, add_bias_kv=True, add_zero_attn=True, batch_first=True)
    x = torch.randn(B, T, E)
    layer = DenseSoftmaxLayer()
    kpm = LengthMask(torch.tensor([4, 2]), max_len=T)
    am = FullMask(torch.tril(torch.ones(T, T, dtype=torch.bool)))
    out, w = m(layer, x, x, x, key_padding_mask=kpm, attn_mask=am, need_weights=True)
    seen_am, seen_kpm = layer.seen
    assert seen_kpm.bool_matrix.shape == (B, T + 2) and seen_kpm.lengths.tolist() == [6, 4]
    assert seen_am.bool_matrix.shape == (T, T + 2) and bool(seen_am.bool_matrix[:, :2].all())
    assert torch.equal(seen_am.bool_matrix[:, 2:], am.bool_matrix)
    assert w.shape == (B, H, T, T + 2) and out.shape == (B, T, E)
    # keys: zero position, bias_k, then the projected keys; masked keys get no weight
    assert float(w[1, :, :, 4:].detach().abs().max()) == 0.0
    with pytest.raises(RuntimeError):
        m(layer, x, x, x, attn_mask=FullMask(torch.ones(T, T + 1, dtype=torch.bool)))
    with pytest.raises(AssertionError):
        m(layer, torch.randn(B, T, E + 1), x, x)


@pytest.mark.gpu
def test_wrapper_around_sblocal_attention_matches_oracle_layer():
    from conftest import rel_err
    from fly_amd import SBLocalAttention
    from oracle import sblocal as osb
    torch.manual_seed(0)
    dev = torch.device('cuda:0')
    E, H, B, T, lc = 128, 2, 2, 320, 64
    mha = MultiheadAttention(E, H, batch_first=True).to(dev)
    attn = SBLocalAttention(local_context=lc, dim_heads=E // H, nb_features=64).to(dev).eval()
    x = torch.randn(B, T, E, device=dev)
    lengths = torch.tensor([320, 190])
    out, w = mha(attn, x, x, x, key_padding_mask=LengthMask(lengths.to(dev), max_len=T))
    assert w is None and out.shape == (B, T, E)

    class OracleLayer(torch.nn.Module):
        def forward(self, q, k, v, attn_mask=None, key_padding_mask=None, need_weights=False):
            P = attn.feature_map.projection_matrix.double().cpu()
            o, _ = osb.sblocal_attention(q.double(), k.double(), v.double(), P, lc,
                                         key_lengths=key_padding_mask.lengths.cpu())
            return o, None

    ref, _ = mha.double().cpu()(OracleLayer(), x.double().cpu(), x.double().cpu(), x.double().cpu(),
                                key_padding_mask=LengthMask(lengths, max_len=T))
    assert rel_err(out.cpu(), ref) <= 1e-4, rel_err(out.cpu(), ref)


@pytest.mark.gpu
def test_wrapper_around_blocksparse_attention_matches_dense_masked_softmax():
    """Seq-first inputs, bias_k / zero position off, a key-padding mask: the wrapper around
    BlockSparseAttention (bf16, fused kernel) against the same wrapper around a plain softmax layer
    restricted to the layout's blocks."""
    from conftest import rel_err
    from fly_amd import BlockSparseAttention
    torch.manual_seed(0)
    dev = torch.device('cuda:0')
    E, H, B, T = 256, 4, 2, 256

    class BandPerHead:
        """One layout per head: a band whose width grows with the head, plus the first block-column."""
        block = 32

        def make_layout(self, seqlen):
            r = torch.arange(seqlen // self.block)
            lay = torch.stack([((r.view(-1, 1) - r.view(1, -1)).abs() <= h).long() for h in range(H)])
            lay[:, :, 0] = 1
            return lay

    mha = MultiheadAttention(E, H).to(dev)
    attn = BlockSparseAttention(BandPerHead(), attention_dropout=0.0, max_seq_length=T).to(dev).eval()
    x = torch.randn(T, B, E, device=dev)
    lengths = torch.tensor([256, 160], device=dev)
    with torch.no_grad():
        out, w = mha.bfloat16()(attn, x.bfloat16(), x.bfloat16(), x.bfloat16(),
                                key_padding_mask=LengthMask(lengths, max_len=T))
    assert w is None and out.shape == (T, B, E)
    dense = attn.get_layout(T).to(dev).bool().repeat_interleave(32, 1).repeat_interleave(32, 2)      # (H, T, T)

    class MaskedLayer(torch.nn.Module):
        def forward(self, q, k, v, attn_mask=None, key_padding_mask=None, need_weights=False):
            s = torch.einsum('bthd,bshd->bhts', q, k) / math.sqrt(q.shape[-1])
            s = s + key_padding_mask.additive_matrix[:, None, None, :]
            s = s.masked_fill(~dense[None], float('-inf'))
            return torch.einsum('bhts,bshd->bthd', s.softmax(dim=-1), v), None

    with torch.no_grad():
        ref, _ = mha.float()(MaskedLayer(), x, x, x, key_padding_mask=LengthMask(lengths, max_len=T))
    assert rel_err(out.float().cpu(), ref.cpu()) <= 3e-2, rel_err(out.float().cpu(), ref.cpu())
