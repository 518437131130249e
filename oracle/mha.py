"""Oracle restatement of the reference's nested multi-head attention.

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

min_mha follows nestedtensor/csrc/mha.cpp:18-69 through the packed fast
paths it dispatches to: NestedTensor_matmul (matmul.cpp:13-41: one GEMM on
``buffer.reshape(-1, E)``), packed add (BinaryOps.cpp:97-107), per-constituent
mul (BinaryOps.cpp:296-299), reshape/transpose (shape.cpp:31-83), per-constituent
softmax (SoftMax.cpp:12-28) and identity dropout when not training
(autograd_functions.cpp:16-22).  Every intermediate is stored in the input
dtype, as ATen does.

bt_min_mha follows nestedtensor/csrc/cuda/mha.cpp:22-107 with the softmax of
nestedtensor/csrc/cuda/attention.cu:229-304: scores over the padded length
with the additive mask ``(1 - m_q m_k) * -10000``, scale applied to the scores,
``exp / (sum + 1e-6)``, and no output bias.
"""

import torch


def _lengths(nt):
    return [int(v) for v in nt.sizes[:, 0]]


def min_mha(num_heads, head_dim, dropout_p, training, query, key, value,
            in_proj_weight, in_proj_bias, scaling, out_proj_weight, out_proj_bias):
    """mha.cpp:18-69.  query/key/value: RefNestedTensor of dim 3 with regular
    last dim E.  Returns the list of per-sequence outputs [L_i, E]."""
    if query.dim() != 3:
        raise RuntimeError("query needs to be 3 dim.")
    if key.dim() != 3:
        raise RuntimeError("key needs to be 3 dim.")
    if value.dim() != 3:
        raise RuntimeError("value needs to be 3 dim.")
    if in_proj_bias is None:
        raise RuntimeError("Input projection bias needs to be defined.")
    assert not training, "dropout is the identity only when not training"
    opt = query.opt_sizes()
    if opt[2] is None:
        raise RuntimeError("query's third dimension must be regular.")
    E = opt[2]
    W = in_proj_weight
    # mha.cpp:42-50 with matmul.cpp:13-41: one packed GEMM each
    q = query.buffer.reshape(-1, E) @ W[0:E].t().contiguous()
    k = key.buffer.reshape(-1, E) @ W[E:2 * E].t().contiguous()
    v = value.buffer.reshape(-1, E) @ W[2 * E:].t().contiguous()
    # mha.cpp:52-54
    q = q + in_proj_bias[0:E].contiguous()
    k = k + in_proj_bias[E:2 * E].contiguous()
    v = v + in_proj_bias[2 * E:].contiguous()
    # mha.cpp:56: q * torch::tensor(scaling) -- a 0-d float32 tensor; type
    # promotion keeps q's dtype.
    q = q * torch.tensor(scaling)
    outs = []
    lq, lk = _lengths(query), _lengths(key)
    oq = ok = 0
    for Lq, Lk in zip(lq, lk):
        # mha.cpp:58-60: reshape to [L, H, hd], transpose -> [H, L, hd]
        qi = q[oq:oq + Lq].reshape(Lq, num_heads, head_dim).transpose(0, 1)
        ki = k[ok:ok + Lk].reshape(Lk, num_heads, head_dim).transpose(0, 1)
        vi = v[ok:ok + Lk].reshape(Lk, num_heads, head_dim).transpose(0, 1)
        w = torch.matmul(qi, ki.transpose(1, 2))          # mha.cpp:61
        w = torch.softmax(w, -1)                          # mha.cpp:62
        o = torch.matmul(w, vi)                           # mha.cpp:64
        o = o.transpose(0, 1).reshape(Lq, E)              # mha.cpp:65
        outs.append(o)
        oq += Lq
        ok += Lk
    packed = torch.cat(outs, 0)
    packed = packed @ out_proj_weight.t()                 # mha.cpp:66
    packed = packed + out_proj_bias                       # mha.cpp:67
    res, off = [], 0
    for L in lq:
        res.append(packed[off:off + L])
        off += L
    return res


def bt_min_mha(num_heads, head_dim, dropout_p, training, query, key, value,
               attr_kernel, attr_bias, scaling, out_proj_weight, out_proj_bias,
               math_dtype=torch.float32):
    """cuda/mha.cpp:22-107 restated on the CPU.  The softmax math runs in
    ``math_dtype`` (the float kernels of attention.cu compute in fp32)."""
    if query.dim() != 3:
        raise RuntimeError("query needs to be 3 dim.")
    E = num_heads * head_dim
    lens = _lengths(query)
    B, Lmax = len(lens), max(lens)
    dtype = query.buffer.dtype
    packed = query.buffer.reshape(-1, E) @ attr_kernel.t() + attr_bias   # :57
    padded = torch.zeros(B, Lmax, 3 * E, dtype=dtype)                    # :59
    off = 0
    for b, L in enumerate(lens):
        padded[b, :L] = packed[off:off + L]
        off += L
    qb, kb, vb = padded.chunk(3, -1)                                     # :60
    qb = qb.reshape(B, Lmax, num_heads, head_dim).transpose(1, 2)
    kb = kb.reshape(B, Lmax, num_heads, head_dim).transpose(1, 2)
    vb = vb.reshape(B, Lmax, num_heads, head_dim).transpose(1, 2)
    scores = torch.matmul(qb, kb.transpose(2, 3)).contiguous()           # :72
    m = torch.zeros(B, Lmax)
    for b, L in enumerate(lens):
        m[b, :L] = 1
    attr_mask = m.view(B, 1, 1, Lmax)
    attr_mask = attr_mask * attr_mask.transpose(2, 3)                    # :76-79
    # attention.cu:229-260
    s = scores.to(math_dtype) * scaling + (1.0 - attr_mask.to(math_dtype)) * -10000.0
    s = s - s.max(-1, keepdim=True).values
    e = torch.exp(s)
    p = (e / (e.sum(-1, keepdim=True) + 1e-6)).to(dtype)
    o = torch.matmul(p, vb)                                              # :103
    o = o.transpose(1, 2).reshape(B, Lmax, E).contiguous()               # :104
    outs = [o[b, :L] for b, L in enumerate(lens)]                        # :105
    packed_o = torch.cat(outs, 0) @ out_proj_weight.t()                  # :106 (no bias)
    res, off = [], 0
    for L in lens:
        res.append(packed_o[off:off + L])
        off += L
    return res
