"""lean_transformer_amd: the LeanFFN hot path of learning-at-home/lean_transformer on hand-written MI355X (gfx950) kernels.

Public surface mirrors the reference's for this path: ``LeanFFN``, ``GeneralizedLinear`` / ``GeneralizedMatrix``, the
block-sparse layout registry and ``ACT2FN``.
"""
from .blocksparse import (GeneralizedLinear, GeneralizedMatrix, blocksparse_matmul, blocksparse_matmul_backward,
                          get_blocksparse_layout, get_indices_from_layout, register_blocksparse_layout)
from .checkpoint import (LEGACY_KEY_RENAMES, block_list_to_native, convert_legacy_state_dict, load_reference_state_dict,
                         native_to_block_list)
from .ffn import LeanFFN
from .utils import ACT2FN

__version__ = "0.1.0"
