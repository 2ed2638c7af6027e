"""MI355X-native Evoformer attention: a torch.autograd.Function over a C-ABI library of
hand-written gfx950 kernels.  Same call surface as lvhoaa/evoformer_triton's
`evoformer.EvoformerAttention`."""
from .evoformer import EvoformerAttention, DS4Sci_EvoformerAttention, evoformer_attention, slot_attention  # noqa: F401

__all__ = ["EvoformerAttention", "DS4Sci_EvoformerAttention", "evoformer_attention", "slot_attention"]
