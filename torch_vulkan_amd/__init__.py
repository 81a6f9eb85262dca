"""MI355X-native quantized matmul behind torch-vulkan's operator API.

``torch_vulkan_amd.abi``   ctypes binding of the C ABI (include/vkt.h)
``torch_vulkan_amd.build`` builds the HIP library in-tree
The PrivateUse1 ("vk") torch backend that registers the aten ops lives in
``torch_vulkan_amd.backend`` and is imported on demand.
"""
from . import abi  # noqa: F401
