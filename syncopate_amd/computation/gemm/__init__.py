from .template import gemm, gemm_consumer, gemm_producer  # noqa: F401
from .template_remote import (  # noqa: F401
    gemm_ag_direct_read,
    gemm_remote,
    gemm_rs_producer_persistent,
    gemm_splitk,
)
from .tile_policy import choose_tile  # noqa: F401
