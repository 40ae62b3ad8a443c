from .compute import HipCompute, Compute
from .core import HipCore, DeviceBuffer
from .fnn import HipFNN
from .attention import HipAttention

__all__ = ["HipCompute", "Compute", "HipCore", "DeviceBuffer", "HipFNN", "HipAttention"]
