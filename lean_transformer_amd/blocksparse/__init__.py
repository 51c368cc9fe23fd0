"""Block-sparse weights for LeanFFN / GeneralizedLinear: layouts (layout.py), the matmul in the reference's "native" weight
format on HIP kernels (native_backend.py) and the parameter containers (linear.py).  The native format needs a balanced
layout (equal number of active blocks in every block row and every block column) and supports any block size."""
from .layout import (REGISTERED_LAYOUTS, get_blocksparse_layout, get_butterfly_layout, get_hypercube_layout,
                     get_indices_from_layout, register_blocksparse_layout)
from .linear import GeneralizedLinear, GeneralizedMatrix, _GeneralizedLinear
from .native_backend import blocksparse_matmul, blocksparse_matmul_backward
