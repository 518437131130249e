"""nestedtensor_amd: the ragged hot path of pytorch/nestedtensor for MI355X.

Same public names as the reference package (nestedtensor/__init__.py:3-22) for
the part that is built: constructors, padding / mask conversions, the
``NestedTensor`` wrapper and the nested multi-head attention hook.  Use it as
``import nestedtensor_amd as nestedtensor``.
"""

from . import _C  # loads libnestedtensor_amd.so; raises ImportError if it is not built
from . import ops  # registers torch.ops.nestedtensor.*

from .nested.creation import as_nested_tensor
from .nested.creation import nested_tensor

from .nested.masking import nested_tensor_from_tensor_mask
from .nested.masking import nested_tensor_from_padded_tensor
from .nested.masking import from_padded_tensor

from .nested.nested import NestedTensor
from .nested.nested import transpose_nchw_nhwc
from .nested.nested import transpose_nhwc_nchw
from .nested.nested import linear_act

from .ops import set_attention_kernel, set_index_check
from .ops import check_index_errors

from . import nested
from . import nn

__version__ = "0.1.0"
