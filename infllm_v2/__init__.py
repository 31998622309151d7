"""Drop-in alias: ``import infllm_v2`` resolves to the MI355X implementation, with the same public
names as the reference package (infllm_v2/__init__.py:1-11) plus ``infllm_v2.C``."""
from infllmv2_cuda_impl_amd import *  # noqa: F401,F403
from infllmv2_cuda_impl_amd import __version__, __all__  # noqa: F401
