from sla_amd.sparse_attn import _attention  # noqa: F401
