"""The operator surface of the reference's Triton sibling (hexa_moe_triton/hexa_moe/kernels): `counter`,
`ESMM` and `es_fused` with its argument lists and list formats -- token ids padded to chunks of 16 per expert
with -1 (0 after the caller's `+ 1`: ids are 1-based for the operators, 0 names a zero pad row), one expert id
per chunk -- over the HIP library's C ABI.  No Triton is involved."""
from .basics import counter  # noqa: F401
from .esmm import ESMM  # noqa: F401
from .fused import es_fused  # noqa: F401
