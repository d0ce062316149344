from .template import gemm, gemm_consumer, gemm_producer  # noqa: F401
