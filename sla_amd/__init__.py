"""MI355X-native Sparse-Linear Attention: HIP kernels behind the reference's operator API."""
from .block_map import get_block_map, mean_pool  # noqa: F401
from .sparse_attn import _attention  # noqa: F401
from .module import SparseLinearAttention  # noqa: F401
from .sage import SageSparseLinearAttention  # noqa: F401
from .dit_block import SLASelfAttention  # noqa: F401
