from sla_amd.sage import SageSparseLinearAttention  # noqa: F401
