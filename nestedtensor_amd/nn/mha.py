"""Nested multi_head_attention_forward (nestedtensor/nn/mha.py:7-83): what
``torch.nn.MultiheadAttention`` reaches through ``NestedTensor.__torch_function__``
when query / key / value are NestedTensors of shape (bsz, tgt_len_i, embed_dim)."""

import torch

from ..nested import nested

# NT case query, key, value have nested_dim 1 and are of shape (bsz, tgt_len, embed_dim)


def multi_head_attention_forward(query,
                                 key,
                                 value,
                                 embed_dim_to_check,
                                 num_heads,
                                 in_proj_weight,
                                 in_proj_bias,
                                 bias_k,
                                 bias_v,
                                 add_zero_attn,
                                 dropout_p,
                                 out_proj_weight,
                                 out_proj_bias,
                                 training=True,
                                 key_padding_mask=None,
                                 need_weights=True,
                                 attn_mask=None,
                                 use_separate_proj_weight=False,
                                 q_proj_weight=None,
                                 k_proj_weight=None,
                                 v_proj_weight=None,
                                 static_k=None,
                                 static_v=None,
                                 average_attn_weights=True,
                                 is_causal=False,
                                 ):
    assert isinstance(query, nested.NestedTensor)
    assert isinstance(key, nested.NestedTensor)
    assert isinstance(value, nested.NestedTensor)
    assert torch.is_tensor(out_proj_weight)
    assert torch.is_tensor(out_proj_bias)

    # Explicitly unsupported flags (nn/mha.py:36-45)
    assert not use_separate_proj_weight
    assert attn_mask is None
    assert key_padding_mask is None
    assert bias_k is None
    assert bias_v is None
    assert static_k is None
    assert static_v is None
    assert not add_zero_attn
    assert not is_causal

    bsz, tgt_len, embed_dim = query.size()
    assert embed_dim == embed_dim_to_check
    # allow MHA to have different sizes for the feature dimension
    assert key.size(0) == value.size(0) and key.size(1) == value.size(1)

    head_dim = embed_dim // num_heads
    assert head_dim * num_heads == embed_dim, "embed_dim must be divisible by num_heads"
    scaling = float(head_dim) ** -0.5

    # The reference sends self-attention with device weights to bt_min_mha, which
    # drops out_proj_bias and is handed in_proj_bias in its place (nn/mha.py:57-69,
    # cuda/mha.cpp:106).  Both branches compute the same function when the biases
    # are zero; here one fused device path serves both and follows min_mha
    # (mha.cpp:18-69), i.e. out_proj_bias is added.
    return torch.ops.nestedtensor.min_mha(num_heads,
                                          head_dim,
                                          dropout_p,
                                          training,
                                          query,
                                          key,
                                          value,
                                          in_proj_weight,
                                          in_proj_bias,
                                          scaling,
                                          out_proj_weight,
                                          out_proj_bias), None
