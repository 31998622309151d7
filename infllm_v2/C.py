"""``infllm_v2.C``: the reference's native-module interface (csrc/entry.cu:197-215), served by the HIP library."""
from infllmv2_cuda_impl_amd.C import *  # noqa: F401,F403
