"""Operator boundary of the packed routed-expert forward.

Same module-level names as the reference (bitsmoe/algorithms/__init__.py:28-47) so that
host code written against it (`from bitsmoe.algorithms import _HAS_MLP_FORWARD_CUDA,
mlp_forward_cuda`) binds unchanged: `mlp_forward_cuda` is the operator module whose
`moe_packed_forward` runs the HIP kernels of libbitsmoe_hip.so.  There is no CPU or
PyTorch fallback: when the library is missing `mlp_forward_cuda` is None and the host
block raises, exactly as the reference does without its extension.
"""
import torch


def get_cuda_device_name() -> str:
    """Human-readable accelerator name, "cpu" when none is visible
    (reference: bitsmoe/algorithms/__init__.py:4-25)."""
    if not torch.cuda.is_available():
        return "cpu"
    props = torch.cuda.get_device_properties(torch.cuda.current_device())
    return f"{props.name.strip()} ({round(props.total_memory / 1024 ** 3)}GB)"


_MLP_FORWARD_IMPORT_ERROR = None
try:
    from bitsmoe_amd.algorithms import _mlp_forward_hip as mlp_forward_cuda

    _HAS_MLP_FORWARD_CUDA = True
    _MLP_FORWARD_BACKEND = get_cuda_device_name()
except Exception as exc:  # library not built / not loadable
    mlp_forward_cuda = None
    _HAS_MLP_FORWARD_CUDA = False
    _MLP_FORWARD_BACKEND = "None"
    _MLP_FORWARD_IMPORT_ERROR = exc

__all__ = [
    "mlp_forward_cuda",
    "_HAS_MLP_FORWARD_CUDA",
    "_MLP_FORWARD_BACKEND",
    "get_cuda_device_name",
]
