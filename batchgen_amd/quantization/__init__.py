"""Host-side mirror of the reference's ``batchgen/quantization`` entry points on the MoE path."""
from .act_quant import act_quant  # noqa: F401
