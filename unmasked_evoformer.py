"""Drop-in module name of the reference's second copy of the operator
(dsevoformer-triton/unmasked_evoformer.py:585 `class EvoformerAttention`): the same maths with
loads and stores that are not predicated, for N_res % 128 == 0 only (:711).  Here one set of
kernels serves every N_res (rows past the end are predicated in the staging, nothing else
branches), so this name is the same operator as `evoformer.EvoformerAttention`."""
from evoformer_triton_amd.evoformer import EvoformerAttention  # noqa: F401
