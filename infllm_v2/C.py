"""``infllm_v2.C``: the reference's native module (csrc/entry.cu:197-215) - here the compiled PyTorch extension
``infllmv2_cuda_impl_amd._C`` (csrc/torch_module.cpp) over the C ABI of the HIP library."""
from infllmv2_cuda_impl_amd._C import *  # noqa: F401,F403
