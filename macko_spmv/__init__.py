"""`import macko_spmv` alias of macko_spmv_amd, so code written against the upstream package
(src/macko_spmv/__init__.py) runs unchanged on MI355X."""
from macko_spmv_amd import (  # noqa: F401
    __compressor_lib,
    __multiply_lib,
    LIB_NAME,
    __version__,
    compress,
    compress_int8,
    decompress,
    move_to_device,
    multiply,
    multiply_axpby,
    multiply_batched,
    multiply_int8,
    multiply_int8_axpby,
    multiply_rmsnorm,
    multiply_silu_mul_axpby,
)
