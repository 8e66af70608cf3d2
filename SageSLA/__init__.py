"""Drop-in import name of the reference's SageSLA package, backed by ``sla_amd.sage``."""
from sla_amd.sage import SageSparseLinearAttention

__all__ = ["SageSparseLinearAttention"]
