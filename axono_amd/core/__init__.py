from .tensor import Tensor, get_default_device, hip_available, set_default_device
from .types import DataType, Status


def cuda_available() -> bool:
    """There is no CUDA path in this build; see hip_available()."""
    return False


__all__ = ["DataType", "Status", "Tensor", "cuda_available", "hip_available", "get_default_device",
           "set_default_device"]
