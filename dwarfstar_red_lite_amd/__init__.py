"""MI355X-native routed-expert MoE FFN behind the reference's redmetal_ffn / redmetal_quant / router call surface.

The arithmetic lives in libredmetal_hip.so (hand-written gfx950 HIP, see csrc/); this package is the host-side
mirror of the reference's ctypes bridges (redlite/redmetal_ffn.py, redlite/redmetal_quant.py) plus the resident
layer API. PyTorch is used only to own device memory and streams.
"""
from ._lib import RedHipError, load  # noqa: F401

TYPE_F32, TYPE_Q6_K, TYPE_IQ2_XXS, TYPE_IQ3_S = 0, 14, 16, 21


def expert_type_word(gate_up_type, down_type):
    """Two-type word of the reference (native/redlite_native_metal.h:69-73)."""
    return gate_up_type | ((down_type << 8) if down_type != gate_up_type else 0)
