"""Packed storage of a nested tensor: buffer + nested size + device offsets.

Counterpart of the reference's NestedTensorImpl / EfficientSizeNode
(nestedtensor/csrc/nested_tensor_impl.h:46-173,
nestedtensor/csrc/storage/EfficientSizeNode.h:53-138): one contiguous 1-D
buffer, a host int64 table ``sizes[B, D]`` and the per-dimension "regular or
not" summary ``opt_sizes``.  What is new here is the device side of the
metadata: ``sizes`` mirrored in HBM and int64 element ``offsets[B + 1]`` built
by the device prefix scan (nt_offsets_from_sizes), both cached on the impl and
created on first use on the buffer's stream.  Only nested_dim 1 exists
(EfficientSizeNode.h:86-88).

Two storage layouts exist, as in the reference (Packed.h:100-163): every
constituent row-major contiguous, or, for constituents [C, H, W], every
constituent stored as [H, W, C] ("channels last", the nested stride is then
(1, W * C, C)).  The second is a flag on the impl, not a stride table: these
are the only two layouts the reference's kernels accept, and the constituent
extents, hence the element offsets, are the same in both.
"""

import torch

from . import _C


class NestedTensorImpl:
    __slots__ = ("buffer", "sizes", "_opt_sizes", "_sizes_dev", "_offsets_dev",
                 "_row_offsets_dev", "_max_sizes", "_attn_schedule", "_attn_plan", "_last_dim_rows", "_has_empty", "_transpose_meta",
                 "channels_last")

    def __init__(self, buffer, sizes, channels_last=False):
        """buffer: 1-D contiguous tensor; sizes: CPU int64 [B, D], or 0-d for an
        empty nested tensor (EfficientSizeNode.h:8-12).  channels_last: the
        buffer holds each [C, H, W] constituent as [H, W, C]."""
        if buffer.dim() != 1:
            raise RuntimeError("Given buffer must be vector, i.e. dim 1 Tensor.")
        if not buffer.is_contiguous():
            raise RuntimeError("Given buffer must be contiguous.")
        assert sizes.dtype == torch.int64 and sizes.device.type == "cpu"
        if channels_last and not (sizes.dim() == 2 and sizes.size(1) == 3):
            raise RuntimeError("ChannelsLast memory format requires 4 dim input.")
        self.channels_last = bool(channels_last)
        self.buffer = buffer
        self.sizes = sizes
        self._opt_sizes = None
        self._sizes_dev = None
        self._offsets_dev = None
        self._row_offsets_dev = None
        self._max_sizes = None
        self._attn_schedule = None
        self._attn_plan = None
        self._last_dim_rows = None
        self._has_empty = None
        self._transpose_meta = None

    # ---- host metadata ----------------------------------------------------
    @property
    def B(self):
        return self.sizes.size(0) if self.sizes.dim() > 0 else 0

    @property
    def D(self):
        return self.sizes.size(1) if self.sizes.dim() > 0 else 0

    def dim(self):
        # EfficientSizeNode::dim (EfficientSizeNode.h:94-96)
        return 1 + self.sizes.size(1) if self.sizes.dim() > 0 else 1

    def nested_dim(self):
        return 1

    def numel(self):
        # EfficientSizeNode::numel (EfficientSizeNode.h:113-131)
        if self.sizes.dim() == 0 or self.sizes.numel() == 0:
            return 0
        return int(self.sizes.prod(1).sum())

    def opt_sizes(self):
        # construct_efficient_size (EfficientSizeNode.h:27-49)
        if self._opt_sizes is None:
            res = [self.B]
            if self.sizes.dim() > 0 and self.B > 0:
                first = self.sizes[0]
                same = (self.sizes == first).all(0)
                for j in range(self.D):
                    res.append(int(first[j]) if bool(same[j]) else None)
            self._opt_sizes = res
        return list(self._opt_sizes)

    def max_sizes(self):
        # get_max_size_from_efficient_size (masking.cpp:83-103)
        if self._max_sizes is None:
            if self.B > 0 and self.D > 0:
                self._max_sizes = [int(v) for v in self.sizes.max(0).values]
            else:
                self._max_sizes = []
        return list(self._max_sizes)

    def has_empty_constituent(self):
        if self._has_empty is None:
            self._has_empty = self.B > 0 and self.D > 0 and bool((self.sizes == 0).any())
        return self._has_empty

    def shapes(self):
        return [tuple(int(v) for v in row) for row in self.sizes] if self.sizes.dim() > 0 else []

    def strides(self):
        """Per-constituent element strides: row-major (Packed.h:10-19), or
        (1, W * C, C) for the channels-last layout (nested_tensor_impl.cpp:188-192)."""
        out = []
        for s in self.shapes():
            if self.channels_last:
                out.append((1, s[2] * s[0], s[0]))
                continue
            st, acc = [], 1
            for v in reversed(s):
                st.append(acc)
                acc *= v
            out.append(tuple(reversed(st)))
        return out

    # ---- device metadata ---------------------------------------------------
    def sizes_dev(self):
        if self._sizes_dev is None:
            _C.require_device(self.buffer, "device metadata")
            self._sizes_dev = self.sizes.contiguous().to(self.buffer.device)
        return self._sizes_dev

    def offsets_dev(self):
        """int64 [B + 1] element offsets, built on the device by the prefix scan."""
        if self._offsets_dev is None:
            self._offsets_dev = device_offsets(self.sizes_dev(), self.B, self.D)
        return self._offsets_dev

    def row_offsets_dev(self):
        """int64 [B + 1] offsets counted in rows of the first constituent dim
        (token offsets for a [B, L_i, E] nested tensor)."""
        if self._row_offsets_dev is None:
            first = self.sizes_dev()[:, :1].contiguous()
            self._row_offsets_dev = device_offsets(first, self.B, 1)
        return self._row_offsets_dev

    def last_dim_rows(self):
        """(row_offsets, total_rows): int64 [B + 1] on the device, the number of
        rows along the last dim (product of all other constituent dims) of the
        constituents before b, and their total."""
        if self._last_dim_rows is None:
            rows = self.sizes[:, :-1].prod(1)
            row_offsets = torch.zeros(self.B + 1, dtype=torch.int64)
            row_offsets[1:] = torch.cumsum(rows, 0)
            self._last_dim_rows = (row_offsets.to(self.buffer.device), int(row_offsets[-1]))
        return self._last_dim_rows

    def attention_schedule(self, kv=None, q_tile=128):
        """Work list of the attention kernel, built from the host copies of the
        nested sizes and cached on the device: int32 [n_work, 8] rows {first query
        token, query length, first query row of the tile, 0, first key token, key
        length, 0, 0}, one per q_tile query rows of every sequence, longest key
        sequences first (they take the most key tiles, so they should start
        first).  Tiles that do not exist are never listed, hence never launched.
        kv: the nested tensor of the keys (None: self-attention)."""
        if kv is None or kv.sizes is self.sizes:
            kv = self
        cached = self._attn_schedule
        if cached is not None and cached[0] is kv.sizes:
            return cached[1]
        q_lens, k_lens = self.sizes[:, 0], kv.sizes[:, 0]
        if int(q_lens.sum()) > 0x7fffffff or int(k_lens.sum()) > 0x7fffffff:
            raise RuntimeError("attention: %d query and %d key tokens; the work list holds token indices "
                               "as int32" % (int(q_lens.sum()), int(k_lens.sum())))
        q_starts = torch.cumsum(q_lens, 0) - q_lens
        k_starts = torch.cumsum(k_lens, 0) - k_lens
        order = torch.argsort(k_lens, descending=True, stable=True)
        ntile = (q_lens[order] + q_tile - 1) // q_tile
        seq = order[torch.repeat_interleave(torch.arange(order.numel()), ntile)]
        first = torch.cumsum(ntile, 0) - ntile
        rank = torch.repeat_interleave(torch.arange(order.numel()), ntile)
        q0 = (torch.arange(int(ntile.sum())) - first[rank]) * q_tile
        zero = torch.zeros_like(q0)
        items = torch.stack([q_starts[seq], q_lens[seq], q0, zero, k_starts[seq], k_lens[seq], zero, zero], 1)
        sched = items.to(torch.int32).contiguous().to(self.buffer.device)
        self._attn_schedule = (kv.sizes, sched)      # holds kv.sizes, so the identity test stays valid
        return sched

    def attention_plan(self, num_heads, head_dim, kv=None):
        """Plan of the planned attention kernel (nt_attention_plan) for this nested
        size, `num_heads` heads and the compute units of the buffer's device: an
        int32 vector on the device, cached like the work list.
        kv: the nested tensor of the keys (None: self-attention)."""
        if kv is None or kv.sizes is self.sizes:
            kv = self
        cached = self._attn_plan
        if cached is not None and cached[0] is kv.sizes and cached[1] == (num_heads, head_dim):
            return cached[2]
        plan = _C.ops.attention_plan.default(self.sizes[:, 0].contiguous(), kv.sizes[:, 0].contiguous(),
                                             num_heads, head_dim, self.buffer.device)
        self._attn_plan = (kv.sizes, (num_heads, head_dim), plan)
        return plan

    def adopt_device_metadata(self, sizes_dev, offsets_dev):
        """Take over device copies of the nested size and of the element offsets
        that a conversion has already built for this nested size."""
        if sizes_dev.device == self.buffer.device and tuple(sizes_dev.shape) == tuple(self.sizes.shape):
            self._sizes_dev = sizes_dev
            if offsets_dev.numel() == self.B + 1:
                self._offsets_dev = offsets_dev

    def with_buffer(self, buffer, channels_last=None):
        """Same nested size over another buffer (in the same layout unless
        channels_last says otherwise); shares the cached metadata when the
        device matches."""
        out = NestedTensorImpl(buffer, self.sizes,
                               self.channels_last if channels_last is None else channels_last)
        out._opt_sizes = self._opt_sizes
        out._max_sizes = self._max_sizes
        out._has_empty = self._has_empty
        if buffer.device == self.buffer.device:
            out._sizes_dev = self._sizes_dev
            out._offsets_dev = self._offsets_dev
            out._row_offsets_dev = self._row_offsets_dev
            out._attn_schedule = self._attn_schedule
            out._attn_plan = self._attn_plan
            out._last_dim_rows = self._last_dim_rows
            out._transpose_meta = self._transpose_meta
        return out


_offsets_from_sizes = _C.ops.offsets_from_sizes.default


def device_offsets(sizes_dev, B, D):
    """offsets[b] = sum_{c<b} prod_k sizes[c, k] on the device (nt_offsets_from_sizes)."""
    return _offsets_from_sizes(sizes_dev.reshape(B, D))
