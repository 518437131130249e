"""CPU oracle for the nestedtensor ragged hot path.  TEST INFRASTRUCTURE ONLY.

This package restates, with plain ``torch`` CPU ops and Python loops, what the
reference's CPU code paths compute for packing, padding, un-padding, masks and
nested multi-head attention.  Every function cites the reference file:line it
follows.  It exists so that the HIP kernels can be checked for parity; nothing
in the shipped package (``nestedtensor_amd``) imports it.  Only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` use it,
and only as the checker / the timed CPU baseline.

The arithmetic below the reference's own code lives in ATen (``at::matmul``,
``at::softmax``, ``at::constant_pad_nd``, ``at::stack``, ``at::masked_select``),
which the reference pins at torch 1.11.0.dev20220202 and which is not vendored
in its tree; the oracle calls the same ATen entry points of the installed
torch.  Padding, un-padding and masks are pure data movement, so their results
do not depend on the ATen version and parity is bit-exact.  Attention parity is
tolerance-based.

Pinning (what each part was checked against, see tests/test_oracle_*.py):

* pack / nested_size / size / nested_stride: literal cases of
  test/test_nested_tensor_class.py:199-231, 256-265, 449-472 and the closed
  form ``buffer == cat(flatten(t_i))``.
* to_tensor_mask / to_mask: literal cases of
  test/test_nested_tensor_masking.py:11-142, ``to_mask == to_tensor_mask()[1]``
  (test/test_nested_tensor_class.py:809-817) and the closed form
  ``mask[b, i...] = all(i_k < size[b, k])``.
* nt_from_tensor_mask: literal cases of
  test/test_nested_tensor_masking.py:146-452.
* to_padded_tensor: literal case of test/test_nested_tensor_masking.py:454-477,
  ``torch.nn.utils.rnn.pad_sequence`` and core ``torch.nested`` as independent
  library cross-checks.
* from_padded_tensor: round trip with to_padded_tensor and ``padded[mask]``.
* min_mha: ``torch.nn.MultiheadAttention`` per sequence (the reference's own
  differential, test/test_nested_tensor_functional.py:648-667) and dense
  attention with ``key_padding_mask`` (:1118-1140), plus an fp64 brute force.
* bt_min_mha: equality with min_mha at 1e-5 for zero out-bias
  (test/test_nested_tensor_functional.py:1115).
* layer_norm (written out in fp64, not a call of torch's): torch's
  ``layer_norm`` per constituent, which is what the reference's test compares
  with (test/test_nested_tensor_functional.py:894-917), and the closed forms
  (zero mean, variance var/(var + eps), shift invariance).
* max_pool2d / conv2d: the per-constituent mapping the reference's tests assert
  (test/test_nested_tensor_functional.py:44-135, 251-266); the output sizes are
  cross-checked against the closed form of pooling.cpp:50-53 / conv2d.cpp:80-84
  in tests/test_oracle_rowops.py.
* embedding / embedding_bag / to_sparse_csr / to_packed_sequence: closed forms
  that avoid the library call being restated (indexing, Python loops, the CSR
  ``to_dense`` check of test/test_nested_tensor_class.py:741-752, the
  ``pad_packed_sequence`` round trip); tests/test_oracle_interop.py.
* to_channels_last / from_channels_last: torch's own
  ``contiguous(memory_format=torch.channels_last)`` per constituent, values and
  strides (test/test_nested_tensor_class.py:844-866), and the round trip.
* softmax: rows sum to 1, invariance to a per-row shift, the closed form
  ``exp(x) / sum(exp(x))`` in fp64 written out with Python loops, and
  ``log_softmax == log(softmax)`` (tests/test_oracle_rowops.py).
* activation: relu against ``max(x, 0)``, gelu against the closed form
  ``x/2 (1 + erf(x / sqrt 2))`` with math.erf in fp64 (tests/test_oracle_rowops.py).
* mul / matmul: per-constituent ``torch.mul`` / ``torch.matmul`` are the
  reference's own definition (BinaryOps.cpp:296-299, matmul.cpp:44-49); pinned
  against hand-computed values and an fp64 product in tests/test_oracle_rowops.py.
* add: ``torch.add`` on the packed buffers / per constituent
  (test/test_nested_tensor_functional.py's add cases reduce to it).

Two reference behaviours are restated here but deliberately not followed by
the product: the uint8-vs-bool mask dtype of merge_tensor_mask
(masking.cpp:149-157, 31) and the double push of 0-d constituents in the CPU
to_padded_tensor (masking.cpp:644-647).
"""

from .nt import RefNestedTensor, ref_nested_tensor  # noqa: F401
from .masking import (  # noqa: F401
    get_max_size,
    merge_tensor_mask,
    pad_tensor_to_shape,
    pad_nt,
    to_tensor_mask,
    to_mask,
    to_padded_tensor,
    from_padded_tensor,
    nt_from_tensor_mask,
    nt_from_tensor_mask_vectorised,
    nested_tensor_from_tensor_mask,
    nested_tensor_from_padded_tensor,
)
from .mha import min_mha, bt_min_mha  # noqa: F401
from .rowops import layer_norm, add, mul, matmul, softmax, activation  # noqa: F401
from .dense import max_pool2d, conv2d  # noqa: F401
from .interop import (  # noqa: F401
    embedding, embedding_bag, to_sparse_csr, to_packed_sequence, transpose_nchw_nhwc, transpose_nhwc_nchw,
    to_channels_last, from_channels_last)
