"""Known-answer cases transcribed (as data) from the reference's own tests,
test/test_nested_tensor_masking.py.  Each entry gives inputs and the expected
result; they pin the oracle on the CPU and are replayed against the HIP path on
the GPU."""

import torch

T = torch.tensor

# to_tensor_mask: (constituents, ctor dtype, [(mask_dim, expected tensor, expected mask)])
# test_nested_tensor_masking.py:11-132
TO_TENSOR_MASK = [
    ("empty_nt", [], None, [(None, T([0]), T(False))]),
    ("single_scalar", [T(1, dtype=torch.uint8)], torch.uint8, [
        (None, T([1], dtype=torch.uint8), T(True)),
        (0, T([1], dtype=torch.uint8), T(True)),
        (1, T([1], dtype=torch.uint8), T([True])),
    ]),
    ("single_tensor", [T([1])], None, [
        (None, T([[1.]]), T(True)),
        (0, T([[1.]]), T(True)),
        (1, T([[1.]]), T([True])),
        (2, T([[1.]]), T([[True]])),
    ]),
    ("multi_tensor", [T([1]), T([2]), T([3])], None, [
        (None, T([[1.], [2.], [3.]]), T(True)),
        (0, T([[1.], [2.], [3.]]), T(True)),
        (1, T([[1.], [2.], [3.]]), T([True, True, True])),
        (2, T([[1.], [2.], [3.]]), T([[True], [True], [True]])),
    ]),
]

# to_tensor_mask errors: (constituents, dtype, mask_dim, message)
# test_nested_tensor_masking.py:19-25, 46-49, 98-101, 134-142
TO_TENSOR_MASK_ERRORS = [
    ([T([])], None, None, "Empty tensors are not yet supported."),
    ([T(1, dtype=torch.uint8)], torch.uint8, 2,
     "Requested mask dimension 2 is bigger than dimension 1 of given NestedTensor."),
    ([T([1])], None, 3,
     "Requested mask dimension 3 is bigger than dimension 2 of given NestedTensor."),
    ([T([1, 2]), T([3, 4, 5, 6])], None, 1,
     "Mask dimension is too small to represent data tensor."),
]

F = torch.float
# nested_tensor_from_tensor_mask: (name, tensor, mask, expected constituents, expected dtype)
# test_nested_tensor_masking.py:157-449.  The expected dtype is what the
# reference's expected nested_tensor(...) literal has (default float32 unless
# the test passes dtype=).
FROM_TENSOR_MASK = [
    ("empty", T([]), T([]), [], F),
    ("empty2", T([[], []]), T([[], []]), [T([]), T([])], F),
    ("empty3", T([0]), T(False), [], F),
    ("single_scalar_mask_false", T([1], dtype=torch.uint8), T(False), [], F),
    ("single_scalar_a", T([1], dtype=F), T(True), [T(1.)], F),
    ("single_scalar_b", T([1], dtype=F), T([True]), [T(1.)], F),
    ("single_scalar_extra_dim", T([[1]], dtype=F), T(True), [T([1.])], F),
    ("multi_scalars_a", T([1, 2, 3]), T(True), [T(1), T(2), T(3)], torch.int64),
    ("multi_scalars_b", T([1, 2, 3]), T([True]), [T(1), T(2), T(3)], torch.int64),
    ("multi_scalars_extra_dim", T([[1, 2, 3]]), T(True), [T([1, 2, 3])], torch.int64),
    ("single_tensor_all_true_a", T([[1]], dtype=F), T(True), [T([1.])], F),
    ("single_tensor_all_true_b", T([[1]], dtype=F), T([True]), [T([1.])], F),
    ("multi_tensor_scalar_true", T([[1], [2], [3]]), T(True), [T([1]), T([2]), T([3])], torch.int64),
    ("multi_tensor_scalar_true_extra", T([[[1]], [[2]], [[3]]]), T(True),
     [T([[1]]), T([[2]]), T([[3]])], torch.int64),
    ("multi_tensor_true_mask3", T([[[1]], [[2]], [[3]]], dtype=F), T([[[True]], [[True]], [[True]]]),
     [T([[1.]]), T([[2.]]), T([[3.]])], F),
    ("multi_tensor_true_mask2", T([[[1]], [[2]], [[3]]], dtype=F), T([[True], [True], [True]]),
     [T([[1.]]), T([[2.]]), T([[3.]])], F),
    ("multi_tensor_true_mask1", T([[[1]], [[2]], [[3]]], dtype=F), T([True, True, True]),
     [T([[1.]]), T([[2.]]), T([[3.]])], F),
    ("multi_tensor_true_mask0", T([[[1]], [[2]], [[3]]], dtype=F), T(True),
     [T([[1.]]), T([[2.]]), T([[3.]])], F),
    ("single_tensor_all_false_a", T([[1]]), T([False]), [], F),
    ("single_tensor_all_false_b", T([[1, 2, 3]]), T([False]), [], F),
    ("multi_tensor_all_false_a", T([[[1], [2], [3]]]), T([False]), [], F),
    ("multi_tensor_all_false_b", T([[[1], [2], [3]]]), T([False, False, False]), [], F),
    ("multi_tensor_all_false_c", T([[[1], [2], [3]]]), T([[False], [False], [False]]),
     [T([], dtype=torch.int64)], torch.int64),
    ("multi_tensor_all_false2", T([[[1], [2], [3]]]), T([[[False], [False], [False]]]),
     [torch.empty((3, 0), dtype=torch.int64)], torch.int64),
    ("multi_scalar_mix", T([1, 2, 3, 4], dtype=F), T([True, False, False, True]), [T(1.), T(4.)], F),
    ("multi_tensor_mix", T([[1], [2], [3], [4]], dtype=F), T([True, False, False, True]),
     [T([1.]), T([4.])], F),
    ("scalar_with_empty_mix", T([[0], [11]], dtype=F), T([False, True]), [T([11.])], F),
    ("multi_tensor_mix_mask", T([[1, 2, 3], [4, 0, 0]], dtype=F),
     T([[True, True, True], [True, False, False]]), [T([1., 2., 3.]), T([4.])], F),
    ("multi_tensor_mix_mask2", T([[[1, 2, 3]], [[4, 0, 0]]], dtype=F),
     T([[[True, True, True]], [[True, False, False]]]), [T([[1., 2., 3.]]), T([[4.]])], F),
]

# nested_tensor_from_tensor_mask errors: (tensor, mask, nested_dim, exception, message or None)
# test_nested_tensor_masking.py:146-155, 170-171, 205-216, 225-229, 270-271, 451-452
FROM_TENSOR_MASK_ERRORS = [
    (T([]), T([]), 0, RuntimeError, "Nested dimension can't be 0."),
    (None, None, 1, RuntimeError, None),
    (T([]), None, 1, RuntimeError, None),
    (T([]), T([]), 2, RuntimeError, None),
    (T([]), T([True]), 1, RuntimeError, "Data tensor can't be emtpy if a mask has values."),
    (T([1]), T([]), 1, RuntimeError, "Mask tensor can't be emtpy if a data tensor has values."),
    (T(1), T(True), 1, RuntimeError, "Can't construct nested tensor from a scalar."),
    (T([1, 2, 3]), T([True]), 2, RuntimeError, None),
    (T([[[1, 2, 3]], [[4, 0, 0]]], dtype=F), T([[[True, True, True]], [[True, False, False]]]), 4,
     RuntimeError, None),
]

# test_to_padded_tensor (test_nested_tensor_masking.py:454-477)
ROUND_TRIP_DATA = T(
    [[[0.8413, 0.7325, 0.0000, 0.0000],
      [0.0000, 0.0000, 0.0000, 0.0000],
      [0.0000, 0.0000, 0.0000, 0.0000]],
     [[0.6334, 0.5473, 0.3273, 0.0564],
      [0.3023, 0.6826, 0.3519, 0.1804],
      [0.8431, 0.1645, 0.1821, 0.9185]]])
ROUND_TRIP_MASK = T(
    [[[True, True, False, False],
      [False, False, False, False],
      [False, False, False, False]],
     [[True, True, True, True],
      [True, True, True, True],
      [True, True, True, True]]])
