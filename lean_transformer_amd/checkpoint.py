"""Loading checkpoints written by the reference's modules, including its older key names, and converting block-sparse
weights between the "native" on-disk order and a block-list order.

A state_dict of the reference's ``LeanFFN`` / ``GeneralizedLinear`` / ``GeneralizedMatrix`` already uses the parameter and
buffer names of this package and loads with ``load_state_dict`` as is.  Checkpoints from before the reference renamed its
submodules need the substitutions its own test applies before loading (tests/test_gpt_exact_match.py:51-80), and they lack
the persistent ``.layout`` buffers, which can be rebuilt from the module's constructor arguments.
"""
from typing import Dict, Mapping, Optional, Tuple

import torch
import torch.nn as nn

# (old substring, new substring), applied in this order to every key
LEGACY_KEY_RENAMES: Tuple[Tuple[str, str], ...] = (
    (".shared_matrix.", ".matrix."),
    (".dense_qkv", ".qkv_proj"),
    (".dense_out", ".out_proj"),
    (".dense_i2h", ".i2h_proj"),
    (".dense_h2o", ".h2o_proj"),
    ("attention.layer_norm", "attention.pre_layer_norm"),
    ("ffn.layer_norm", "ffn.pre_layer_norm"),
    (".sandwich_norm", ".post_layer_norm"),
)


def convert_legacy_state_dict(state: Mapping[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    """The same tensors under today's key names.  Keys are matched with a leading "." where the rename table has one, so a
    state_dict of a bare FFN block (keys like ``dense_i2h.weight``) is handled by matching against "." + key."""
    out = {}
    for key, value in state.items():
        dotted = "." + key
        for old, new in LEGACY_KEY_RENAMES:
            dotted = dotted.replace(old, new)
        new_key = dotted[1:]
        if new_key in out:
            raise KeyError(f"legacy keys collide after renaming: {new_key!r}")
        out[new_key] = value
    return out


def load_reference_state_dict(module: nn.Module, state: Mapping[str, torch.Tensor], strict: bool = True):
    """``module.load_state_dict`` for a checkpoint in the reference's format, current or legacy.

    Applies ``LEGACY_KEY_RENAMES`` and fills in buffers that older checkpoints did not store but that follow from how
    ``module`` was constructed: ``*.layout`` and, where absent, the ``*.forward_indices`` / ``*.backward_indices`` tables.
    Tensors are copied into the module's existing parameters (their dtype and device are kept).  Shape mismatches and, with
    ``strict``, missing or unexpected keys raise as in ``load_state_dict``; returns its report."""
    converted = convert_legacy_state_dict(state)
    own = module.state_dict()
    rebuilt = (".layout", ".forward_indices", ".backward_indices")
    for key, value in own.items():
        if key not in converted and key.endswith(rebuilt):
            converted[key] = value
    for key in own:
        if key.endswith((".forward_indices", ".backward_indices")) and key in converted:
            if converted[key].shape != own[key].shape or not torch.equal(converted[key].to(own[key]), own[key]):
                raise ValueError(
                    f"{key} of the checkpoint differs from the table this module built from its layout descriptor: the "
                    "checkpoint was written for another block layout (its weight blocks would be applied in the wrong places)")
    return module.load_state_dict(converted, strict=strict)


def native_to_block_list(weight: torch.Tensor, backward_indices: torch.Tensor, out_features: int
                         ) -> Tuple[torch.Tensor, torch.Tensor]:
    """Native block-sparse weight ``[in_features, A, block]`` -> (blocks ``[nnz, block, block]``, coords ``[nnz, 2]``).

    Block ``n`` is the dense sub-matrix ``W[ob * block : (ob + 1) * block, ib * block : (ib + 1) * block]`` (rows = output
    features, columns = input features) with ``coords[n] = (ob, ib)``, listed in row-major order of the layout (ascending
    output block, then ascending input block): the order a block list built from ``layout.nonzero()`` has.  The native
    tensor read as ``[in_blocks, A, block, block]`` holds the same sub-matrices ordered by input block, then by the rank of
    the output block among that input block's active blocks (lean_transformer/blocksparse/native_backend.py:24-27)."""
    in_features, per_in, block = weight.shape
    in_blocks = in_features // block
    if backward_indices.shape != (in_blocks, per_in):
        raise ValueError(f"backward_indices {tuple(backward_indices.shape)} does not match weight {tuple(weight.shape)}")
    blocks = weight.reshape(in_blocks, per_in, block, block)
    ob = backward_indices.to(torch.int64).reshape(-1)
    ib = torch.arange(in_blocks, device=ob.device).repeat_interleave(per_in)
    if int(ob.max()) >= out_features // block:
        raise ValueError("backward_indices names an output block past out_features")
    order = torch.argsort(ob * in_blocks + ib)
    coords = torch.stack([ob[order], ib[order]], dim=1)
    return blocks.reshape(in_blocks * per_in, block, block)[order.to(weight.device)].contiguous(), coords


def block_list_to_native(blocks: torch.Tensor, coords: torch.Tensor, backward_indices: torch.Tensor) -> torch.Tensor:
    """Inverse of ``native_to_block_list``: places block ``n`` (for output block ``coords[n, 0]``, input block
    ``coords[n, 1]``) at its slot of the native ``[in_features, A, block]`` tensor that ``backward_indices`` describes."""
    in_blocks, per_in = backward_indices.shape
    nnz, block, _ = blocks.shape
    if nnz != in_blocks * per_in:
        raise ValueError(f"{nnz} blocks given, the layout has {in_blocks * per_in}")
    table: Dict[Tuple[int, int], int] = {}
    bi = backward_indices.to(torch.int64).cpu()
    for ib in range(in_blocks):
        for a in range(per_in):
            table[(int(bi[ib, a]), ib)] = ib * per_in + a
    slots = torch.empty(nnz, dtype=torch.int64)
    for n, (ob, ib) in enumerate(coords.cpu().tolist()):
        try:
            slots[n] = table[(ob, ib)]
        except KeyError:
            raise ValueError(f"block {n} at (output block {ob}, input block {ib}) is not active in this layout") from None
    if slots.unique().numel() != nnz:
        raise ValueError("two blocks of the list name the same position")
    native = torch.empty_like(blocks)
    native[slots.to(blocks.device)] = blocks
    return native.reshape(in_blocks, per_in, block, block).reshape(in_blocks * block, per_in, block)
