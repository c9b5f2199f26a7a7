"""Import alias: `from ncn_cuda_amd.ncn_pytorch_wrapper_v2 import NCNNetCuda` works like the reference's module path
(ncn_cuda/ncn_pytorch_wrapper_v2.py); the classes live in ncn_cuda_amd/modules.py."""
from .modules import *  # noqa: F401,F403
from .modules import __all__  # noqa: F401
