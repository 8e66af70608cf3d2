from sla_amd.block_map import get_block_map, mean_pool  # noqa: F401
