"""Drop-in mirror of the reference's ``mix_moe`` Python package for one MI355X.

Same module, class and function names as the reference
(mix_moe/mix_moe/{transformer,layers,linear,functions}.py and gates/), backed by
the HIP library through ``ccfuser_amd.ops``.  One GPU only: ``world_size`` must
be 1 and nothing here opens a communicator.
"""
from .gates import BaseGate, NaiveGate
from .layers import MixMOE
from .linear import FMoELinear, MixMOEInstance, MixMOELinear1, MixMOELinear2
from .transformer import AsyncExpertAssignment, MixMOETransformerMLP

__all__ = ["BaseGate", "NaiveGate", "MixMOE", "FMoELinear", "MixMOEInstance", "MixMOELinear1",
           "MixMOELinear2", "AsyncExpertAssignment", "MixMOETransformerMLP"]
