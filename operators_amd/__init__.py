"""operators_amd - host-side Python mirror of the InfiniOperators harness for
the MI355X `amd-gpu` device (Add, RMSNorm, RoPE, SwiGLU).

Plays the role of the reference's `operatorspy` package: load libinfiniop.so,
describe torch tensors to it and call the C entry points.  All arithmetic is
done by the library's HIP kernels; there is no Python or CPU implementation
behind these names.
"""
from .data_layout import *  # noqa: F401,F403
from .devices import DeviceEnum  # noqa: F401
from .liboperators import (  # noqa: F401
    CTensor,
    infiniopAddDescriptor_t,
    infiniopAddRMSNormDescriptor_t,
    infiniopAttentionDescriptor_t,
    infiniopCausalSoftmaxDescriptor_t,
    infiniopHandle_t,
    infiniopMatmulDescriptor_t,
    infiniopMLPDescriptor_t,
    infiniopRearrangeDescriptor_t,
    infiniopRMSNormDescriptor_t,
    infiniopRandomSampleDescriptor_t,
    infiniopRoPEDescriptor_t,
    infiniopSwiGLUDescriptor_t,
    infiniopTensorDescriptor_t,
    open_lib,
)
from .utils import (  # noqa: F401
    InfiniopError,
    check_error,
    create_handle,
    create_workspace,
    destroy_handle,
    destroy_tensor,
    make_descriptor,
    rearrange_tensor,
    to_tensor,
)
