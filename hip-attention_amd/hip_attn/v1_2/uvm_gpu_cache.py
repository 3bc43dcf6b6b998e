"""Alias module: the reference keeps the offload cache classes in ``hip_attn.v1_2.uvm_gpu_cache``."""
from ..offload import GPUCache, HiPOffloadCache, UVMCache  # noqa: F401
