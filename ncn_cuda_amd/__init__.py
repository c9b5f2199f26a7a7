"""MI355X (gfx950) implementation of the NCN layer behind the reference's Python surface."""
from . import ncn_cuda_module
from .modules import (ACTIVATION_CODES, NCNFunction, NCNModuleCuda, NCNNetCuda, NCNNetFunction,
                                     NCNNetTestCuda, NCNRadixNetFunction, default_save_every, fused_ncn_cuda_v2, fused_ncn_net,
                      fused_ncn_radix_net, ncn_inverse)

__all__ = ["ncn_cuda_module", "ACTIVATION_CODES", "NCNFunction", "NCNModuleCuda", "NCNNetCuda", "NCNNetTestCuda",
           "fused_ncn_cuda_v2", "ncn_inverse", "NCNNetFunction", "fused_ncn_net", "default_save_every",
           "NCNRadixNetFunction", "fused_ncn_radix_net"]
