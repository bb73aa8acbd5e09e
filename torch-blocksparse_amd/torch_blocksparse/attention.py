"""nn.MultiheadAttention with a block-sparse attention pattern.

Drop-in for the reference's torch_blocksparse/attention.py: `MultiheadAttention(embed_dim, num_heads, layout,
block, ...)`, `multi_head_attention_forward`, `replace_mha`, `make_layout`.  The projections stay dense PyTorch;
the score / softmax / context product are the block-sparse operators.  Unlike the reference, the operator
cache belongs to the module (attention.py:207-218 caches per sequence length on the class, across layouts),
and `replace_mha` passes the block size it forgot (attention.py:272).
"""
import torch
import torch.nn as nn
from torch.nn.functional import linear

from .attention_core import attention_chain
from .layouts import make_layout  # noqa: F401  (re-exported like the reference's attention.make_layout)
from .matmul import MatMul
from .softmax import Softmax


def multi_head_attention_forward(query, key, value, embed_dim_to_check, num_heads, in_proj_weight, in_proj_bias,
                                 bias_k, bias_v, add_zero_attn, dropout_p, out_proj_weight, out_proj_bias,
                                 sparse_dot_sdd_nt, sparse_dot_dsd_nn, sparse_softmax, training=True,
                                 key_padding_mask=None, need_weights=True, attn_mask=None,
                                 use_separate_proj_weight=False, q_proj_weight=None, k_proj_weight=None,
                                 v_proj_weight=None, static_k=None, static_v=None, key_padding_mask_mode='add',
                                 attn_mask_mode='add', key_block_pad=0):
    """Same signature and result as the reference (attention.py:9-202): returns (attn_output, None).

    bias_k / bias_v and add_zero_attn append one key position each, as in nn.functional.multi_head_attention_forward; the
    masks grow by columns that leave those positions visible (0 in 'add' mode, 1 in 'mul' mode).  key_block_pad more
    zero positions are then appended and hidden through the key-padding mask (one is made if the caller passed none), so
    that the keys fill a whole number of blocks; the sparse operators passed in must be built on a layout with the
    matching number of block-columns (MultiheadAttention does both)."""
    tgt_len, bsz, embed_dim = query.size()
    assert embed_dim == embed_dim_to_check
    assert key.size() == value.size()
    head_dim = embed_dim // num_heads
    assert head_dim * num_heads == embed_dim, 'embed_dim must be divisible by num_heads'
    scaling = float(head_dim) ** -0.5

    def bias_slice(lo, hi):
        return None if in_proj_bias is None else in_proj_bias[lo:hi]

    E = embed_dim
    if not use_separate_proj_weight:
        if (query is key or torch.equal(query, key)) and (key is value or torch.equal(key, value)):
            q, k, v = linear(query, in_proj_weight, in_proj_bias).chunk(3, dim=-1)
        elif key is value or torch.equal(key, value):
            q = linear(query, in_proj_weight[:E], bias_slice(0, E))
            k, v = linear(key, in_proj_weight[E:], bias_slice(E, None)).chunk(2, dim=-1)
        else:
            q = linear(query, in_proj_weight[:E], bias_slice(0, E))
            k = linear(key, in_proj_weight[E:2 * E], bias_slice(E, 2 * E))
            v = linear(value, in_proj_weight[2 * E:], bias_slice(2 * E, None))
    else:
        assert q_proj_weight.shape == (E, query.size(-1))
        assert k_proj_weight.shape == (E, key.size(-1))
        assert v_proj_weight.shape == (E, value.size(-1))
        q = linear(query, q_proj_weight, bias_slice(0, E))
        k = linear(key, k_proj_weight, bias_slice(E, 2 * E))
        v = linear(value, v_proj_weight, bias_slice(2 * E, None))
    q = q * scaling                                      # attention.py:127, so softmax runs with scale 1

    def grow(mask, n, mode, visible=True):
        if mask is None:
            return None
        shown, hidden = (0., float('-inf')) if mode == 'add' else (1., 0.)
        return torch.cat([mask, mask.new_full((mask.size(0), n), shown if visible else hidden)], dim=1)

    if bias_k is not None and bias_v is not None:
        assert static_k is None and static_v is None, 'bias cannot be added to static key/value.'
        k = torch.cat([k, bias_k.repeat(1, bsz, 1)])
        v = torch.cat([v, bias_v.repeat(1, bsz, 1)])
        attn_mask, key_padding_mask = grow(attn_mask, 1, attn_mask_mode), grow(key_padding_mask, 1, key_padding_mask_mode)
    else:
        assert bias_k is None and bias_v is None

    q = q.contiguous().view(tgt_len, bsz * num_heads, head_dim).transpose(0, 1)
    k = k.contiguous().view(-1, bsz * num_heads, head_dim).transpose(0, 1)
    v = v.contiguous().view(-1, bsz * num_heads, head_dim).transpose(0, 1)
    if static_k is not None:
        assert static_k.size(0) == bsz * num_heads and static_k.size(2) == head_dim
        k = static_k
    if static_v is not None:
        assert static_v.size(0) == bsz * num_heads and static_v.size(2) == head_dim
        v = static_v
    src_len = k.size(1)
    if key_padding_mask is not None:
        assert key_padding_mask.size(0) == bsz and key_padding_mask.size(1) == src_len
    if attn_mask is not None:
        assert attn_mask.size(0) == tgt_len and attn_mask.size(1) == src_len
    if add_zero_attn:
        src_len += 1
        k = torch.cat([k, k.new_zeros((k.size(0), 1) + k.size()[2:])], dim=1)
        v = torch.cat([v, v.new_zeros((v.size(0), 1) + v.size()[2:])], dim=1)
        attn_mask, key_padding_mask = grow(attn_mask, 1, attn_mask_mode), grow(key_padding_mask, 1, key_padding_mask_mode)
    if key_block_pad:
        k = torch.cat([k, k.new_zeros((k.size(0), key_block_pad) + k.size()[2:])], dim=1)
        v = torch.cat([v, v.new_zeros((v.size(0), key_block_pad) + v.size()[2:])], dim=1)
        if key_padding_mask is None:
            key_padding_mask = q.new_full((bsz, src_len), 0. if key_padding_mask_mode == 'add' else 1.)
        key_padding_mask = grow(key_padding_mask, key_block_pad, key_padding_mask_mode, visible=False)
        attn_mask = grow(attn_mask, key_block_pad, attn_mask_mode)
        src_len += key_block_pad

    q = q.reshape(bsz, num_heads, q.shape[1], q.shape[2]).contiguous()
    k = k.reshape(bsz, num_heads, k.shape[1], k.shape[2]).contiguous()
    v = v.reshape(bsz, num_heads, v.shape[1], v.shape[2]).contiguous()
    # The reference's three calls (attention.py:190-202), in one launch where the kernels allow it.  Dropout on the
    # attention weights (nn.functional.multi_head_attention_forward applies it after the softmax; the reference raises
    # NotImplementedError for dropout != 0) is fused into the softmax kernel of the three-operator path.
    out = attention_chain(sparse_dot_sdd_nt, sparse_softmax, sparse_dot_dsd_nn, q, k, v, key_padding_mask=key_padding_mask,
                          attn_mask=attn_mask, key_padding_mask_mode=key_padding_mask_mode, attn_mask_mode=attn_mask_mode,
                          dropout_p=float(dropout_p) if training else 0.)
    out = out.reshape(bsz * num_heads, out.shape[2], out.shape[3])
    out = out.transpose(0, 1).contiguous().view(tgt_len, bsz, embed_dim)
    out = linear(out, out_proj_weight, out_proj_bias)
    return out, None


class MultiheadAttention(nn.modules.activation.MultiheadAttention):

    def extra_keys(self):
        """Key positions appended to the sequence: one for bias_k / bias_v, one for add_zero_attn."""
        return int(self.bias_k is not None) + int(bool(self.add_zero_attn))

    def get_ops(self, L):
        if L not in self._ops:
            layout = self.layout
            if self.extra_keys():
                # The appended positions get a block-column of their own, present in every block-row of every head
                # (nn.MultiheadAttention shows them to every query); the rest of that block is padding, hidden through
                # the key-padding mask.  The reference accepts the two flags and then runs its kernels on a key length
                # that is not a whole number of blocks (attention.py:140-186).
                layout = torch.cat([layout, torch.ones_like(layout[:, :, :1])], dim=2)
            self._ops[L] = (MatMul(layout, self.block, 'sdd', trans_a=False, trans_b=True),
                            MatMul(layout, self.block, 'dsd', trans_a=False, trans_b=False),
                            Softmax(layout, self.block))
        return self._ops[L]

    def __init__(self, embed_dim, num_heads, layout, block, dropout=0., bias=True, add_bias_kv=False, add_zero_attn=False,
                 kdim=None, vdim=None, key_padding_mask_mode='add', attn_mask_mode='mul'):
        super(MultiheadAttention, self).__init__(embed_dim, num_heads, dropout, bias, add_bias_kv, add_zero_attn, kdim, vdim)
        self.layout = layout
        self.block = block
        self.key_padding_mask_mode = key_padding_mask_mode
        self.attn_mask_mode = attn_mask_mode
        self._ops = dict()

    def forward(self, query, key, value, key_padding_mask=None, need_weights=True, attn_mask=None,
                average_attn_weights=True, is_causal=False):
        """query / key / value: [L, batch, embed] ([batch, L, embed] if the module was made batch_first by replace_mha).
        The last two arguments exist because current torch.nn layers pass them; attention weights are never returned
        (the second result is None, as in the reference) and is_causal without a mask is refused."""
        if query.shape != key.shape or key.shape != value.shape:
            raise NotImplementedError('only self-attention is supported for now')
        if is_causal and attn_mask is None:
            raise NotImplementedError('is_causal needs the causal mask passed as attn_mask (or a causal layout)')
        if self.batch_first:
            query, key, value = [t.transpose(0, 1) for t in (query, key, value)]
        sdd_nt, dsd_nn, softmax = self.get_ops(query.shape[0])
        extra = dict()
        if self.extra_keys():
            extra['key_block_pad'] = self.block - self.extra_keys()
        if not self._qkv_same_embed_dim:
            extra.update(use_separate_proj_weight=True, q_proj_weight=self.q_proj_weight,
                         k_proj_weight=self.k_proj_weight, v_proj_weight=self.v_proj_weight)
        out, _ = multi_head_attention_forward(
            query, key, value, self.embed_dim, self.num_heads, self.in_proj_weight, self.in_proj_bias,
            self.bias_k, self.bias_v, self.add_zero_attn, self.dropout, self.out_proj.weight, self.out_proj.bias,
            sdd_nt, dsd_nn, softmax, training=self.training, key_padding_mask=key_padding_mask,
            need_weights=need_weights, attn_mask=attn_mask, key_padding_mask_mode=self.key_padding_mask_mode,
            attn_mask_mode=self.attn_mask_mode, **extra)
        return (out.transpose(0, 1) if self.batch_first else out), None


def _layout_and_block(info, block):
    """(layout, block) from either calling form of replace_mha: (layout, block), or one `info` carrying both: an
    object with attributes `layout` and `block`, a mapping with those keys, or a (layout, block) pair."""
    if block is not None:
        return info, block
    if isinstance(info, dict):
        return info['layout'], info['block']
    if hasattr(info, 'layout') and hasattr(info, 'block'):
        return info.layout, info.block
    if isinstance(info, (tuple, list)) and len(info) == 2:
        return info[0], info[1]
    raise TypeError('replace_mha(model, info): info must carry `layout` and `block` (attributes, keys or a pair); '
                    'or call replace_mha(model, layout, block)')


def replace_mha(model, layout, block=None):
    """Swap every nn.MultiheadAttention inside `model` for the block-sparse one, keeping its parameters, dtype, device
    and batch_first setting.  Two calling forms: replace_mha(model, layout, block), and the reference's
    replace_mha(model, info) (attention.py:267-281), where `info` carries the layout and the block size (the reference
    hands `info` to a constructor that needs both and cannot run as written).  Like the reference it builds the
    replacement with key_padding_mask_mode='mul' and attn_mask_mode='add', the conventions of
    nn.MultiheadAttention's masks (boolean / 0-1 padding mask, additive float attention mask); masks must have the
    dtype of the activations."""
    layout, block = _layout_and_block(layout, block)
    for child_name, child in model.named_children():
        if isinstance(child, nn.modules.activation.MultiheadAttention) and not isinstance(child, MultiheadAttention):
            ref = child.in_proj_weight if child.in_proj_weight is not None else child.q_proj_weight
            mha = MultiheadAttention(child.embed_dim, child.num_heads, layout, block, dropout=child.dropout,
                                     bias=child.in_proj_bias is not None, add_bias_kv=child.bias_k is not None,
                                     add_zero_attn=child.add_zero_attn, kdim=child.kdim, vdim=child.vdim,
                                     key_padding_mask_mode='mul', attn_mask_mode='add').to(device=ref.device, dtype=ref.dtype)
            mha.batch_first = child.batch_first
            mha.load_state_dict(child.state_dict())
            mha.train(child.training)
            setattr(model, child_name, mha)
        else:
            replace_mha(child, layout, block)
