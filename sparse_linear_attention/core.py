from sla_amd.module import SparseLinearAttention  # noqa: F401
