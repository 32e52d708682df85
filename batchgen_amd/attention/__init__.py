from .add_rmsnorm_fp8_quant import cuda_add_rmsnorm_fp8_quant  # noqa: F401
