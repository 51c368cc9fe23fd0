"""CPU oracle (test infrastructure only): block-sparse layouts, index tables and the block-sparse matmul.

Restates lean_transformer/blocksparse/layout.py:56-211 and lean_transformer/blocksparse/native_backend.py:9-76
with explicit index arithmetic (numpy for the integer parts, one einsum per block for the float parts).
"""
import math
from typing import Optional, Tuple

import numpy as np
import torch


def butterfly_mask(size: int, n_factors: int) -> np.ndarray:
    """Boolean [size, size] support of a sum of butterfly factors with strides 1, 2, .., 2**(n_factors-1).

    reference: layout.py:90-91 sums butterfly_factor_to_matrix(ones, k) (layout.py:156-174) for k < n_factors; factor k
    couples index i with i and i ^ 2**k, so the support is {i == j} U {i ^ j == 2**k, k < n_factors}.
    """
    idx = np.arange(size)
    xor = idx[:, None] ^ idx[None, :]
    mask = xor == 0
    for k in range(n_factors):
        mask |= xor == (1 << k)
    return mask


def pixelfly_layout(out_features: int, in_features: int, block_size: int = 256, butterfly_size: Optional[int] = None,
                    n_factors: Optional[int] = None, stretch: bool = False) -> np.ndarray:
    """Boolean [out_features // block_size, in_features // block_size] block mask of the "pixelfly" layout.

    reference: get_butterfly_layout, layout.py:56-117.  Brute force over elements: element (o, i) is active when
    butterfly cell (o // (out/size), i // (in/size)) is; a block is active when any of its elements is
    (layout.py:93-108); without stretch the stretched copies are regrouped into tiled copies (layout.py:109-116).
    """
    if butterfly_size is None:
        butterfly_size = 2 ** int(math.ceil(math.log2(min(in_features, out_features) / block_size)))
    assert out_features % in_features == 0 or in_features % out_features == 0
    assert out_features % block_size == 0 and in_features % block_size == 0
    log_n = int(math.log2(butterfly_size))
    n_factors = log_n if n_factors is None else n_factors
    if butterfly_size != 2 ** log_n or butterfly_size < 2:
        raise NotImplementedError("butterfly_size must be a power of 2")
    if not (1 <= n_factors <= log_n):
        raise NotImplementedError("n_factors must be a between 1 and log_2(butterfly_size)")
    bf = butterfly_mask(butterfly_size, n_factors)
    rows_per_cell, cols_per_cell = out_features // butterfly_size, in_features // butterfly_size
    cell_of_row = np.arange(out_features) // rows_per_cell
    cell_of_col = np.arange(in_features) // cols_per_cell
    n_out, n_in = out_features // block_size, in_features // block_size
    layout = np.zeros((n_out, n_in), dtype=bool)
    for p in range(n_out):
        rows = np.unique(cell_of_row[p * block_size:(p + 1) * block_size])
        for q in range(n_in):
            cols = np.unique(cell_of_col[q * block_size:(q + 1) * block_size])
            layout[p, q] = bf[np.ix_(rows, cols)].any()
    if not stretch:
        if n_out > n_in:
            ratio = n_out // n_in
            layout = layout.reshape(n_out // ratio, ratio, n_in).transpose(1, 0, 2).reshape(n_out, n_in)
        elif n_out < n_in:
            ratio = n_in // n_out
            layout = layout.reshape(n_out, n_in // ratio, ratio).transpose(0, 2, 1).reshape(n_out, n_in)
    return np.ascontiguousarray(layout)


def hypercube_layout(out_features: int, in_features: int, block_size: int, stretch: bool = False,
                     folded: bool = False) -> np.ndarray:
    """reference: get_hypercube_layout, layout.py:120-153: square pixelfly over the smaller dimension, optionally with the
    antipodal edge (index ^ all-ones), then repeated (tiled) or stretched (each cell repeated in place) to the full shape."""
    smaller = min(out_features, in_features)
    assert math.log2(smaller / block_size).is_integer()
    assert out_features % smaller == 0 and in_features % smaller == 0
    dim = int(math.ceil(math.log2(smaller / block_size)))
    layout = pixelfly_layout(smaller, smaller, block_size, n_factors=dim, stretch=False).copy()
    assert layout.shape == (2 ** dim, 2 ** dim)
    if folded:
        for i in range(2 ** dim):
            layout[i, (2 ** dim - 1) ^ i] = True
    ro, ri = out_features // smaller, in_features // smaller
    if stretch:
        layout = np.repeat(np.repeat(layout, ro, axis=0), ri, axis=1)
    else:
        layout = np.tile(layout, (ro, ri))
    return np.ascontiguousarray(layout)


def indices_from_layout(layout: np.ndarray) -> Tuple[np.ndarray, np.ndarray]:
    """(forward_indices int32 [n_out, K], backward_indices int64 [n_in, A]) for a balanced block mask.

    reference: get_indices_from_layout, layout.py:177-211.  backward_indices[ib, a] is the a-th active output block of input
    block ib (ascending); forward_indices[ob, k] = ib * A + a where ib is the k-th active input block of output block ob
    (ascending) and a is the position of ob inside backward_indices[ib].
    """
    n_out, n_in = layout.shape
    per_out = np.unique(layout.sum(1))
    per_in = np.unique(layout.sum(0))
    assert len(per_out) == 1 and len(per_in) == 1, "layout must be balanced"
    K, A = int(per_out[0]), int(per_in[0])
    backward = np.zeros((n_in, A), dtype=np.int64)
    for ib in range(n_in):
        backward[ib] = np.nonzero(layout[:, ib])[0]
    forward = np.zeros((n_out, K), dtype=np.int32)
    for ob in range(n_out):
        for k, ib in enumerate(np.nonzero(layout[ob])[0]):
            a = int(np.nonzero(backward[ib] == ob)[0][0])
            forward[ob, k] = ib * A + a
    return forward, backward


def sparse_to_dense(weight: torch.Tensor, backward_indices, out_features: int) -> torch.Tensor:
    """Dense [out_features, in_features] matrix equal to a native-format sparse weight.

    The parameter is declared [in_features, A, block] (linear.py:48-49) but the matmul reads its memory as
    [n_in_blocks, A, block(out row), block(in col)] (native_backend.py:24: weight.view(num_input_blocks, -1, block_size)),
    and block (ib, a) lands at output block backward_indices[ib, a].
    """
    in_features, A, b = weight.shape
    n_in = in_features // b
    w4 = weight.reshape(n_in, A, b, b)
    bwd = np.asarray(backward_indices)
    dense = torch.zeros(out_features, in_features, dtype=weight.dtype)
    for ib in range(n_in):
        for a in range(A):
            ob = int(bwd[ib, a])
            dense[ob * b:(ob + 1) * b, ib * b:(ib + 1) * b] = w4[ib, a]
    return dense


def blocksparse_matmul(x: torch.Tensor, weight: torch.Tensor, forward_indices) -> torch.Tensor:
    """y[..., ob*b + r] = sum_k sum_c W4[ib_k, a_k, r, c] * x[..., ib_k*b + c], forward_indices[ob, k] = ib_k*A + a_k.

    reference: blocksparse_matmul, native_backend.py:9-35 (per-input-block matmul, then embedding_bag sum per output block).
    """
    in_features, A, b = weight.shape
    n_in = in_features // b
    fwd = np.asarray(forward_indices)
    n_out, K = fwd.shape
    w4 = weight.reshape(n_in, A, b, b)
    x2 = x.reshape(-1, in_features)
    y = torch.zeros(x2.shape[0], n_out * b, dtype=x.dtype)
    for ob in range(n_out):
        for k in range(K):
            ib, a = divmod(int(fwd[ob, k]), A)
            y[:, ob * b:(ob + 1) * b] += torch.einsum("rc,tc->tr", w4[ib, a], x2[:, ib * b:(ib + 1) * b])
    return y.reshape(*x.shape[:-1], n_out * b)


def blocksparse_matmul_backward(dy: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, backward_indices):
    """(dx, dw): dx[t, ib*b+c] = sum_{a,r} W4[ib,a,r,c] dy[t, ob*b+r];  dW4[ib,a,r,c] = sum_t dy[t, ob*b+r] x[t, ib*b+c],
    ob = backward_indices[ib, a].  reference: blocksparse_matmul_backward, native_backend.py:38-76."""
    in_features, A, b = weight.shape
    n_in = in_features // b
    bwd = np.asarray(backward_indices)
    w4 = weight.reshape(n_in, A, b, b)
    x2 = x.reshape(-1, in_features)
    dy2 = dy.reshape(x2.shape[0], -1)
    dx = torch.zeros_like(x2)
    dw4 = torch.zeros_like(w4)
    for ib in range(n_in):
        for a in range(A):
            ob = int(bwd[ib, a])
            g = dy2[:, ob * b:(ob + 1) * b]
            dx[:, ib * b:(ib + 1) * b] += torch.einsum("rc,tr->tc", w4[ib, a], g)
            dw4[ib, a] = torch.einsum("tr,tc->rc", g, x2[:, ib * b:(ib + 1) * b])
    return dx.reshape(x.shape), dw4.reshape(weight.shape)
