"""Block-sparse layouts and the index tables the block-sparse kernels walk (host side, set-up time).

Same registry / descriptor-string interface as the reference (lean_transformer/blocksparse/layout.py:12-53).  The pixelfly
mask is computed at block granularity from the butterfly's closed form instead of through an [out_features, in_features]
element mask, so a 32768 x 4096 layout costs a 512 x 64 table rather than a 134 M-element temporary.
"""
import ast
import logging
import math
from typing import Optional, Tuple

import numpy as np
import torch

logger = logging.getLogger(__name__)
REGISTERED_LAYOUTS = dict()


def register_blocksparse_layout(name: str):
    """Decorator: make ``name(...)`` usable in layout descriptor strings; reference: layout.py:15-21."""
    def _register(f: callable):
        if name in REGISTERED_LAYOUTS:
            logger.warning(f"Overwriting layout {name} with {f}.")
        REGISTERED_LAYOUTS[name] = f
        return f
    return _register


def get_blocksparse_layout(out_features: int, in_features: int, layout: str) -> torch.BoolTensor:
    """Boolean [out_blocks, in_blocks] incidence matrix from a descriptor such as ``pixelfly(block_size=64, stretch=True)``;
    positional and keyword arguments are forwarded to the registered layout function.  reference: layout.py:24-53."""
    assert '(' in layout and layout.endswith(')'), "descriptor format must be name(foo=123, bar='456')"
    parsed = ast.parse(layout).body[0].value
    name = parsed.func.id
    args = [ast.literal_eval(arg) for arg in parsed.args]
    kwargs = {arg.arg: ast.literal_eval(arg.value) for arg in parsed.keywords}
    if name not in REGISTERED_LAYOUTS:
        raise ValueError(f"Unknown layout name {name}, supported layouts: {tuple(REGISTERED_LAYOUTS.keys())}")
    return REGISTERED_LAYOUTS[name](out_features, in_features, *args, **kwargs)


def _butterfly_support(size: int, n_factors: int) -> np.ndarray:
    """support of sum_k factor_k: i == j, or i and j differ in exactly bit k for one k < n_factors"""
    xor = np.bitwise_xor.outer(np.arange(size), np.arange(size))
    ok = xor == 0
    for k in range(n_factors):
        ok |= xor == (1 << k)
    return ok


def _any_over_ranges(mask: np.ndarray, row_lo, row_hi, col_lo, col_hi) -> np.ndarray:
    """out[p, q] = mask[row_lo[p]:row_hi[p]+1, col_lo[q]:col_hi[q]+1].any(), via a 2-D prefix sum"""
    prefix = np.zeros((mask.shape[0] + 1, mask.shape[1] + 1), dtype=np.int64)
    prefix[1:, 1:] = mask.astype(np.int64).cumsum(0).cumsum(1)
    r0, r1 = row_lo[:, None], row_hi[:, None] + 1
    c0, c1 = col_lo[None, :], col_hi[None, :] + 1
    return (prefix[r1, c1] - prefix[r0, c1] - prefix[r1, c0] + prefix[r0, c0]) > 0


@register_blocksparse_layout("pixelfly")
def get_butterfly_layout(out_features: int, in_features: int, block_size: int = 256, butterfly_size: Optional[int] = None,
                         n_factors: Optional[int] = None, stretch: bool = False) -> torch.BoolTensor:
    """Sum of block butterfly factors (https://arxiv.org/abs/2112.00029), without the low-rank term.

    Same arguments and result as the reference's get_butterfly_layout (layout.py:56-117): a butterfly of ``butterfly_size``
    cells is stretched over the matrix, a block is active when it overlaps an active cell, and unless ``stretch`` the
    stretched copies along the longer side are regrouped into tiled copies of the square pattern.
    """
    if butterfly_size is None:
        butterfly_size = 2 ** int(math.ceil(math.log2(min(in_features, out_features) / block_size)))
    assert out_features % in_features == 0 or in_features % out_features == 0, \
        "if matrix is not square, the longer dimension must be a multiple of the shorter dimension"
    assert out_features % block_size == 0 and in_features % block_size == 0
    log_n = int(math.log2(butterfly_size))
    n_factors = log_n if n_factors is None else n_factors
    if butterfly_size != 2 ** log_n or butterfly_size < 2:
        raise NotImplementedError("butterfly_size must be a power of 2")
    if not (1 <= n_factors <= log_n):
        raise NotImplementedError("n_factors must be a between 1 and log_2(butterfly_size)")
    assert out_features % butterfly_size == 0 and in_features % butterfly_size == 0
    support = _butterfly_support(butterfly_size, n_factors)
    rows_per_cell, cols_per_cell = out_features // butterfly_size, in_features // butterfly_size
    n_out, n_in = out_features // block_size, in_features // block_size
    p, q = np.arange(n_out), np.arange(n_in)
    layout = _any_over_ranges(support,
                              (p * block_size) // rows_per_cell, ((p + 1) * block_size - 1) // rows_per_cell,
                              (q * block_size) // cols_per_cell, ((q + 1) * block_size - 1) // cols_per_cell)
    if not stretch:
        if n_out > n_in:
            ratio = n_out // n_in
            layout = layout.reshape(n_out // ratio, ratio, n_in).transpose(1, 0, 2).reshape(n_out, n_in)
        elif n_out < n_in:
            ratio = n_in // n_out
            layout = layout.reshape(n_out, n_in // ratio, ratio).transpose(0, 2, 1).reshape(n_out, n_in)
    return torch.from_numpy(np.ascontiguousarray(layout))


@register_blocksparse_layout("hypercube")
def get_hypercube_layout(out_features: int, in_features: int, block_size: int, stretch: bool = False,
                         folded: bool = False) -> torch.BoolTensor:
    """Pixelfly seen as a hypercube graph, optionally "folded" (an extra edge between antipodal nodes), tiled or stretched
    to a non-square shape.  reference: get_hypercube_layout, layout.py:120-153."""
    smaller = min(out_features, in_features)
    assert math.log2(smaller / block_size).is_integer(), "layout dimension must be a power of 2"
    assert out_features % smaller == 0 and in_features % smaller == 0
    dim = int(math.ceil(math.log2(smaller / block_size)))
    layout = get_butterfly_layout(smaller, smaller, block_size, n_factors=dim, stretch=False).numpy().copy()
    assert layout.shape == (2 ** dim, 2 ** dim)
    if folded:
        nodes = np.arange(2 ** dim)
        assert not layout[nodes, (2 ** dim - 1) ^ nodes].any()
        layout[nodes, (2 ** dim - 1) ^ nodes] = True
    ro, ri = out_features // smaller, in_features // smaller
    layout = np.repeat(np.repeat(layout, ro, axis=0), ri, axis=1) if stretch else np.tile(layout, (ro, ri))
    return torch.from_numpy(np.ascontiguousarray(layout))


def get_indices_from_layout(layout: torch.BoolTensor) -> Tuple[torch.IntTensor, torch.LongTensor]:
    """(forward_indices int32 [out_blocks, K], backward_indices int64 [in_blocks, A]) of a balanced layout.

    backward_indices[ib, a]: a-th active output block of input block ib.  forward_indices[ob, k] = ib * A + a: the flat
    position, in the weight's [in_blocks, A] grid of blocks, of the k-th block that contributes to output block ob.
    reference: get_indices_from_layout, layout.py:177-211 (same dtypes).
    """
    lay = layout.cpu().numpy().astype(bool)
    n_out, n_in = lay.shape
    per_out, per_in = np.unique(lay.sum(1)), np.unique(lay.sum(0))
    assert len(per_out) == 1, "butterfly layout must have the same number of blocks per row"
    assert len(per_in) == 1, "butterfly layout must have the same number of blocks per column"
    K, A = int(per_out[0]), int(per_in[0])
    out_of_in = np.nonzero(lay.T)[1].reshape(n_in, A)  # ascending output blocks of each input block
    in_of_out = np.nonzero(lay)[1].reshape(n_out, K)  # ascending input blocks of each output block
    # rank of output block ob among the active outputs of input block ib = number of active rows above ob in column ib
    rank_in_column = lay.cumsum(0) - 1
    slot = rank_in_column[np.arange(n_out)[:, None], in_of_out]
    forward = in_of_out * A + slot
    return torch.from_numpy(forward.astype(np.int32)), torch.from_numpy(out_of_in.astype(np.int64))
