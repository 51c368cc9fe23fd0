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
    """Decorator that files a layout function ``f(out_features, in_features, *args, **kwargs) -> BoolTensor`` under
    ``name`` so that descriptor strings can call it (same registry as lean_transformer/blocksparse/layout.py:15-21)."""
    def decorator(layout_fn: callable):
        previous = REGISTERED_LAYOUTS.get(name)
        if previous is not None and previous is not layout_fn:
            logger.warning("layout %r was %s and is now %s", name, previous, layout_fn)
        REGISTERED_LAYOUTS[name] = layout_fn
        return layout_fn
    return decorator


def get_blocksparse_layout(out_features: int, in_features: int, layout: str) -> torch.BoolTensor:
    """Boolean [out_blocks, in_blocks] incidence matrix from a descriptor such as ``pixelfly(block_size=64, stretch=True)``:
    a call expression whose literal positional and keyword arguments go to the registered layout function after the two
    sizes.  reference: layout.py:24-53."""
    try:
        call = ast.parse(layout.strip(), mode="eval").body
    except SyntaxError as e:
        raise AssertionError(f"layout descriptor {layout!r} is not of the form name(arg, key=value)") from e
    if not isinstance(call, ast.Call) or not isinstance(call.func, ast.Name):
        raise AssertionError(f"layout descriptor {layout!r} is not of the form name(arg, key=value)")
    make = REGISTERED_LAYOUTS.get(call.func.id)
    if make is None:
        raise ValueError(f"no layout called {call.func.id!r}; registered: {sorted(REGISTERED_LAYOUTS)}")
    positional = [ast.literal_eval(node) for node in call.args]
    named = {kw.arg: ast.literal_eval(kw.value) for kw in call.keywords}
    return make(out_features, in_features, *positional, **named)


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
    longer, shorter = max(out_features, in_features), min(out_features, in_features)
    if longer % shorter:
        raise AssertionError(f"a {out_features} x {in_features} matrix: the longer side must be a multiple of the shorter")
    if out_features % block_size or in_features % block_size:
        raise AssertionError(f"block_size {block_size} does not divide {out_features} x {in_features}")
    if butterfly_size is None:
        butterfly_size = 1 << max(0, math.ceil(math.log2(shorter / block_size)))
    log_n = butterfly_size.bit_length() - 1
    if butterfly_size < 2 or butterfly_size != 1 << log_n:
        raise NotImplementedError(f"butterfly_size {butterfly_size}: a power of two >= 2 is required")
    if n_factors is None:
        n_factors = log_n
    if not 1 <= n_factors <= log_n:
        raise NotImplementedError(f"n_factors {n_factors} outside 1 .. log2(butterfly_size) = {log_n}")
    if out_features % butterfly_size or in_features % butterfly_size:
        raise AssertionError(f"butterfly_size {butterfly_size} does not divide {out_features} x {in_features}")
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
    cells = smaller // block_size
    if smaller % block_size or cells < 1 or cells & (cells - 1):
        raise AssertionError(f"hypercube layout: min(out, in) / block_size = {smaller / block_size} must be a power of two")
    if out_features % smaller or in_features % smaller:
        raise AssertionError("hypercube layout: the longer side must be a multiple of the shorter")
    dim = cells.bit_length() - 1
    layout = get_butterfly_layout(smaller, smaller, block_size, n_factors=dim, stretch=False).numpy().copy()
    if folded:
        nodes = np.arange(cells)
        layout[nodes, (cells - 1) ^ nodes] = True  # antipodal node: all dim bits flipped (not an edge of the plain cube)
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
    if len(per_out) != 1 or len(per_in) != 1:
        raise AssertionError("unbalanced layout: every block row and every block column must hold the same number of active "
                             f"blocks (rows hold {per_out.tolist()}, columns {per_in.tolist()})")
    K, A = int(per_out[0]), int(per_in[0])
    out_of_in = np.nonzero(lay.T)[1].reshape(n_in, A)  # ascending output blocks of each input block
    in_of_out = np.nonzero(lay)[1].reshape(n_out, K)  # ascending input blocks of each output block
    # rank of output block ob among the active outputs of input block ib = number of active rows above ob in column ib
    rank_in_column = lay.cumsum(0) - 1
    slot = rank_in_column[np.arange(n_out)[:, None], in_of_out]
    forward = in_of_out * A + slot
    return torch.from_numpy(forward.astype(np.int32)), torch.from_numpy(out_of_in.astype(np.int64))
