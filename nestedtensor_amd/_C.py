"""ctypes binding of libnestedtensor_amd.so (the C ABI of include/nestedtensor_amd.h).

Plays the role of the reference's compiled module ``nestedtensor._C``
(nestedtensor/csrc/py_init.cpp:218-276): the Python layer reaches native code
only through this module.  There is no fallback: if the shared library is not
built, importing the package fails.
"""

import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libnestedtensor_amd.so")

NT_OK = 0
NT_F32, NT_F16, NT_BF16 = 0, 1, 2
ELEM_TYPE = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2, torch.float64: 3, torch.int8: 4,
             torch.uint8: 5, torch.int16: 6, torch.int32: 7, torch.int64: 8}

_c_void_p = ctypes.c_void_p
_i64 = ctypes.c_int64
_int = ctypes.c_int
_u64 = ctypes.c_uint64
_size_t = ctypes.c_size_t
_f32 = ctypes.c_float
_f64 = ctypes.c_double

# name -> (restype, argtypes); must list every symbol of include/nestedtensor_amd.h
SIGNATURES = {
    "nt_abi_version": (_int, []),
    "nt_last_error": (ctypes.c_char_p, []),
    "nt_offsets_workspace_bytes": (_size_t, [_i64]),
    "nt_offsets_from_sizes": (_int, [_c_void_p, _i64, _i64, _c_void_p, _c_void_p, _size_t, _c_void_p]),
    "nt_offsets_noalloc_max_count": (_i64, []),
    "nt_offsets_from_sizes_noalloc": (_int, [_c_void_p, _i64, _i64, _c_void_p, _c_void_p]),
    "nt_add_padding": (_int, [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _i64, _i64, _i64,
                              ctypes.POINTER(_i64), _int, _u64, _c_void_p]),
    "nt_add_padding_mask": (_int, [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _i64, _i64, _i64,
                                   ctypes.POINTER(_i64), _int, _u64, _c_void_p]),
    "nt_remove_padding": (_int, [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _i64, _i64, _i64,
                                 ctypes.POINTER(_i64), _int, _c_void_p]),
    "nt_build_mask": (_int, [_c_void_p, _c_void_p, _i64, _i64, _i64, ctypes.POINTER(_i64), _c_void_p]),
    "nt_pack": (_int, [_c_void_p, _c_void_p, _c_void_p, _i64, _int, _c_void_p]),
    "nt_pack_table_max_entries": (_i64, []),
    "nt_pack_table": (_int, [_c_void_p, _i64, _i64, _c_void_p, _c_void_p, _int, _c_void_p]),
    "nt_upload_table": (_int, [_c_void_p, _i64, _c_void_p, _c_void_p]),
    "nt_mask_row_counts": (_int, [_c_void_p, _i64, _i64, _c_void_p, _c_void_p, _c_void_p]),
    "nt_leading_boxes_max_dims": (_i64, []),
    "nt_leading_boxes": (_int, [_c_void_p, _c_void_p, _i64, _i64, _c_void_p, _i64, _c_void_p, _c_void_p, ctypes.c_uint32,
                                _c_void_p, _c_void_p]),
    "nt_leading_boxes_stamped": (_int, [_c_void_p, _c_void_p, _i64, _i64, _c_void_p, _i64, _c_void_p, ctypes.c_uint32,
                                        _c_void_p]),
    "nt_value_row_counts": (_int, [_c_void_p, _int, ctypes.c_double, _i64, _i64, _c_void_p, _c_void_p,
                                   _c_void_p]),
    "nt_compact_rows": (_int, [_c_void_p, _c_void_p, _c_void_p, _i64, _i64, _i64, _c_void_p, _c_void_p]),
    "nt_scan_workspace_bytes": (_size_t, [_i64]),
    "nt_exclusive_scan_i32": (_int, [_c_void_p, _i64, _c_void_p, _c_void_p, _size_t, _c_void_p]),
    "nt_linear": (_int, [_c_void_p, _i64, _c_void_p, _c_void_p, _c_void_p, _i64, _i64, _i64, _i64,
                         _int, _c_void_p]),
    "nt_linear_act": (_int, [_c_void_p, _i64, _c_void_p, _c_void_p, _c_void_p, _i64, _i64, _i64, _i64,
                             _int, _int, _c_void_p]),
    "nt_linear_qkv": (_int, [_c_void_p, _i64, _c_void_p, _c_void_p, _c_void_p, _i64, _c_void_p, _i64, _i64,
                             _i64, _i64, _int, _c_void_p]),
    "nt_linear_kv": (_int, [_c_void_p, _i64, _c_void_p, _c_void_p, _c_void_p, _i64, _c_void_p, _i64, _i64,
                            _i64, _i64, _int, _c_void_p]),
    "nt_linear_transposed": (_int, [_c_void_p, _i64, _c_void_p, _c_void_p, _c_void_p, _i64, _i64, _i64, _i64,
                                    _int, _c_void_p]),
    "nt_varlen_attention_vt": (_int, [_c_void_p, _i64, _c_void_p, _i64, _c_void_p, _i64, _c_void_p, _i64,
                                      _c_void_p, _i64, _i64, _i64, _i64, _f32, _int, _c_void_p]),
    "nt_attention_plan": (_i64, [_c_void_p, _c_void_p, _i64, _i64, _i64, _i64, _c_void_p, _i64]),
    "nt_varlen_attention_planned": (_int, [_c_void_p, _i64, _c_void_p, _i64, _c_void_p, _i64, _c_void_p, _i64,
                                           _c_void_p, _i64, _i64, _i64, _i64, _f32, _int, _c_void_p]),
    "nt_varlen_attention_scheduled": (_int, [_c_void_p, _i64, _c_void_p, _i64, _c_void_p, _i64, _c_void_p, _i64,
                                             _c_void_p, _i64, _i64, _i64, _f32, _int, _c_void_p]),
    "nt_varlen_attention": (_int, [_c_void_p, _i64, _c_void_p, _i64, _c_void_p, _i64, _c_void_p, _i64,
                                   _c_void_p, _c_void_p, _i64, _i64, _i64, _i64, _f32, _int,
                                   _c_void_p]),
    "nt_layer_norm": (_int, [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _i64, _i64, _f64, _int,
                             _c_void_p]),
    "nt_add_packed": (_int, [_c_void_p, _c_void_p, _f64, _c_void_p, _i64, _i64, _int, _c_void_p]),
    "nt_softmax_rows": (_int, [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _i64, _i64, _int, _int, _c_void_p]),
    "nt_activation_packed": (_int, [_c_void_p, _c_void_p, _i64, _int, _int, _c_void_p]),
    "nt_mul_packed": (_int, [_c_void_p, _c_void_p, _f64, _c_void_p, _i64, _i64, _int, _c_void_p]),
    "nt_gather_rows": (_int, [_c_void_p, _i64, _i64, _c_void_p, _c_void_p, _i64, _c_void_p, _c_void_p]),
    "nt_packed_sequence_index": (_int, [_c_void_p, _c_void_p, _c_void_p, _i64, _i64, _c_void_p, _c_void_p]),
    "nt_ragged_arange": (_int, [_c_void_p, _i64, _i64, _c_void_p, _c_void_p]),
    "nt_transpose_ragged": (_int, [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _i64, _i64,
                                   _int, _int, _int, _c_void_p]),
    "nt_transpose_ragged_lines": (_int, [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _i64, _i64,
                                         _int, _c_void_p]),
    "nt_conv1x1_tile_pixels": (_i64, []),
    "nt_conv1x1_supported": (_int, [_i64, _i64, _int]),
    "nt_conv1x1_nchw": (_int, [_c_void_p, _c_void_p, _c_void_p, _c_void_p, _c_void_p, _i64, _i64, _i64, _i64, _int,
                               _c_void_p]),
    "nt_embedding_bag": (_int, [_c_void_p, _i64, _i64, _c_void_p, _i64, _c_void_p, _c_void_p, _i64, _i64, _int,
                                _int, _c_void_p, _c_void_p]),
}


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "nestedtensor_amd: %s is missing. Build it with `make -C %s` "
            "(or __graft_entry__.build()); there is no fallback path."
            % (LIB_PATH, os.path.join(_HERE, "csrc")))
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.restype = res
        fn.argtypes = args
    if lib.nt_abi_version() != 1:
        raise ImportError("nestedtensor_amd: ABI version mismatch")
    return lib


lib = _load()

OPS_PATH = os.path.join(_HERE, "_torch_ops.so")


def _load_ops():
    """The operator layer: the C++ torch extension that registers the
    ``nestedtensor`` operator library (csrc/torch_ops.cpp).  No fallback either."""
    if not os.path.exists(OPS_PATH):
        raise ImportError(
            "nestedtensor_amd: %s is missing. Build it with `make -C %s` "
            "(or __graft_entry__.build()); there is no fallback path."
            % (OPS_PATH, os.path.join(_HERE, "csrc")))
    torch.ops.load_library(OPS_PATH)
    return torch.ops.nestedtensor


ops = _load_ops()


def check(rc):
    if rc != NT_OK:
        msg = lib.nt_last_error()
        raise RuntimeError("nestedtensor_amd: %s (code %d)" % (msg.decode() if msg else "error", rc))


def ptr(t):
    """Device (or host) address of a tensor's first element, or None."""
    if t is None:
        return None
    return ctypes.c_void_p(t.data_ptr())


class _NoContext:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_CONTEXT = _NoContext()


def on_device(device):
    """Context that makes `device` the current HIP device for the launches inside
    it; free when it already is (the usual case: one GPU per process)."""
    if device.index is None or device.index == torch.cuda.current_device():
        return _NO_CONTEXT
    return torch.cuda.device(device)


def current_stream(device):
    """hipStream_t of torch's current stream on `device`, as void*."""
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def i64_array(values):
    return (ctypes.c_int64 * max(len(values), 1))(*values)


def dtype_code(dtype):
    if dtype == torch.float32:
        return NT_F32
    if dtype == torch.float16:
        return NT_F16
    if dtype == torch.bfloat16:
        return NT_BF16
    raise RuntimeError("nestedtensor_amd: dtype %s is not supported by this op" % dtype)


def staging_device(what):
    """The device that host (CPU) nested tensors are staged through: the current
    HIP device.  There is no host implementation of the path; without a GPU the
    conversion fails here."""
    if not torch.cuda.is_available():
        raise RuntimeError(
            "nestedtensor_amd: %s of a host tensor is staged through the HIP device, "
            "and no device is visible." % what)
    return torch.device("cuda", torch.cuda.current_device())


def require_device(t, what):
    if not t.is_cuda:
        raise RuntimeError(
            "nestedtensor_amd: %s runs on the HIP device only; got a tensor on %s. "
            "Move the nested tensor with .to('cuda') first." % (what, t.device))
