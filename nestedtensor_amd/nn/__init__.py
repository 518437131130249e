from .mha import multi_head_attention_forward
