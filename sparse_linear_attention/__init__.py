"""Drop-in import name of the reference package, backed by the gfx950 kernels in ``sla_amd``."""
from sla_amd.module import SparseLinearAttention

__all__ = ["SparseLinearAttention"]
