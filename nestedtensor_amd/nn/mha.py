"""Nested multi_head_attention_forward (nestedtensor/nn/mha.py:7-83): what
``torch.nn.MultiheadAttention`` reaches through ``NestedTensor.__torch_function__``
when query / key / value are NestedTensors of shape (bsz, tgt_len_i, embed_dim)."""

import torch

from ..nested import nested

# keyword options of torch.nn.functional.multi_head_attention_forward and the only
# value each may have here (nn/mha.py:36-45 asserts the same set, plus is_causal,
# which torch has grown since); need_weights, training and average_attn_weights are
# accepted as they come: no attention weights are ever returned
_ONLY_VALUE = {
    "use_separate_proj_weight": False, "attn_mask": None, "key_padding_mask": None, "static_k": None,
    "static_v": None, "is_causal": False, "q_proj_weight": None, "k_proj_weight": None, "v_proj_weight": None,
}
_IGNORED = ("need_weights", "training", "average_attn_weights")


def multi_head_attention_forward(query, key, value, embed_dim_to_check, num_heads, in_proj_weight,
                                 in_proj_bias, bias_k, bias_v, add_zero_attn, dropout_p, out_proj_weight,
                                 out_proj_bias, training=True, **options):
    """Returns ``(attention output as a NestedTensor, None)``."""
    for name, operand in (("query", query), ("key", key), ("value", value)):
        assert isinstance(operand, nested.NestedTensor), "%s must be a NestedTensor" % name
    for name, operand in (("out_proj_weight", out_proj_weight), ("out_proj_bias", out_proj_bias)):
        assert torch.is_tensor(operand), "%s must be a Tensor" % name
    assert bias_k is None and bias_v is None and not add_zero_attn, \
        "bias_k, bias_v and add_zero_attn are not supported for NestedTensors"
    for name, given in options.items():
        if name in _IGNORED:
            continue
        assert name in _ONLY_VALUE, "unexpected argument %r" % name
        wanted = _ONLY_VALUE[name]
        assert (given is None) if wanted is None else (not given), \
            "%s=%r is not supported for NestedTensors" % (name, given)

    embed_dim = query.size()[2]
    assert embed_dim == embed_dim_to_check
    # key and value may differ from query in everything but the batch and, between
    # themselves, the sequence lengths
    assert key.size(0) == value.size(0) and key.size(1) == value.size(1)
    head_dim, rest = divmod(embed_dim, num_heads)
    assert rest == 0, "embed_dim must be divisible by num_heads"

    # The reference sends self-attention with device weights to bt_min_mha, which
    # drops out_proj_bias and is handed in_proj_bias in its place (nn/mha.py:57-69,
    # cuda/mha.cpp:106).  Both branches compute the same function when the biases
    # are zero; here one fused device path serves both and follows min_mha
    # (mha.cpp:18-69), i.e. out_proj_bias is added.
    out = torch.ops.nestedtensor.min_mha(
        num_heads, head_dim, dropout_p, training, query, key, value, in_proj_weight, in_proj_bias,
        float(head_dim) ** -0.5, out_proj_weight, out_proj_bias)
    return out, None
