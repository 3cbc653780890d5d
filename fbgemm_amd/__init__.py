"""fbgemm_amd: MI355X (gfx950) implementation of FBGEMM's quantized
embedding-bag hot path (fused row-wise 8-bit / 4-bit / 2-bit pooled lookups and
the table-batched inference forward), behind the reference's operator
interface. See include/fbgemm_amd.h for the C ABI everything goes through."""
from ._lib import LIB_PATH, SYMBOLS, lib  # noqa: F401

FP32, FP16, INT8, INT4, INT2, BF16 = 0, 1, 2, 3, 4, 5
POOL_SUM, POOL_MEAN, POOL_NONE = 0, 1, 2
