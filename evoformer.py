"""Drop-in module name of the reference: `from evoformer import EvoformerAttention`
(dsevoformer-triton/test.py:2, speed_benchmark.py:4, memory_benchmark.py:3)."""
from evoformer_triton_amd.evoformer import EvoformerAttention, DS4Sci_EvoformerAttention  # noqa: F401
