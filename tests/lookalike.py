"""Stand-ins for the reference's modules, written without any class of lean_transformer_amd (test infrastructure).

The reference's tests load a state_dict from a look-alike module into LeanFFN (tests/test_ffn.py:45,199).  These classes
hold parameters and buffers under the reference's names (lean_transformer/ffn.py:51-64,
lean_transformer/blocksparse/linear.py:32-66,109-123), build their layout and index tables with the oracle, and compute with
stock PyTorch ops through the oracle's dense expansion of the block-sparse weight, so autograd differentiates them."""
import math
from typing import Optional

import numpy as np
import torch
import torch.nn as nn
import torch.nn.functional as F

from oracle import blocksparse as obs
from oracle import ffn as offn


class LookAlikeMatrix(nn.Module):
    def __init__(self, in_features, out_features, block_size: Optional[int] = None, lowrank_dim: int = 0, stretch=False):
        super().__init__()
        self.in_features, self.out_features = in_features, out_features
        std = math.sqrt(2.0 / (5 * min(in_features, out_features)))
        if block_size:
            layout = obs.pixelfly_layout(out_features, in_features, block_size, stretch=stretch)
            forward, backward = obs.indices_from_layout(layout)
            self.register_buffer("layout", torch.from_numpy(np.ascontiguousarray(layout)).bool())
            self.register_buffer("forward_indices", torch.from_numpy(np.asarray(forward)).to(torch.int32))
            self.register_buffer("backward_indices", torch.from_numpy(np.asarray(backward)).to(torch.int64))
            self.weight = nn.Parameter(torch.randn(in_features, backward.shape[1], block_size) * std)
        else:
            self.layout = self.forward_indices = self.backward_indices = None
            self.weight = nn.Parameter(torch.randn(out_features, in_features) * std)
        self.lowrank_first = nn.Parameter(torch.randn(lowrank_dim, in_features) * std) if lowrank_dim else None
        self.lowrank_second = nn.Parameter(torch.randn(out_features, lowrank_dim) * std) if lowrank_dim else None

    def dense(self) -> torch.Tensor:
        if self.layout is None:
            return self.weight
        in_features, per_in, block = self.weight.shape
        blocks = self.weight.reshape(in_features // block, per_in, block, block)
        rows = []
        bwd = self.backward_indices.cpu().numpy()
        dense = torch.zeros(self.out_features // block, in_features // block, block, block, dtype=self.weight.dtype,
                            device=self.weight.device)
        ib = torch.arange(in_features // block)[:, None].expand(-1, per_in)
        dense = dense.index_put((torch.from_numpy(bwd), ib), blocks)
        del rows
        return dense.permute(0, 2, 1, 3).reshape(self.out_features, in_features)


class LookAlikeLinear(nn.Module):
    def __init__(self, matrix: LookAlikeMatrix, adapter_dim: int = 0):
        super().__init__()
        self.matrix = matrix
        self.in_features, self.out_features = matrix.in_features, matrix.out_features
        self.bias = nn.Parameter(torch.randn(self.out_features) * 0.1)
        self.adapter_first = nn.Parameter(torch.randn(adapter_dim, self.in_features) * 0.05) if adapter_dim else None
        self.adapter_second = nn.Parameter(torch.randn(self.out_features, adapter_dim) * 0.05) if adapter_dim else None

    def forward(self, x):
        y = F.linear(x, self.matrix.dense(), self.bias)
        if self.matrix.lowrank_first is not None:
            y = y + F.linear(F.linear(x, self.matrix.lowrank_first), self.matrix.lowrank_second)
        if self.adapter_first is not None:
            y = y + F.linear(F.linear(x, self.adapter_first), self.adapter_second)
        return y


class LookAlikeFFN(nn.Module):
    """pre-LN -> i2h -> (gated) tanh GELU -> h2o -> [post-LN] -> + input, as stock ops"""

    def __init__(self, hidden, inter, gated, i2h_proj, h2o_proj, post_layer_norm=False, eps=1e-5):
        super().__init__()
        self.i2h_proj, self.h2o_proj, self.gated = i2h_proj, h2o_proj, gated
        self.pre_layer_norm = nn.LayerNorm(hidden, eps=eps)
        self.post_layer_norm = nn.LayerNorm(hidden, eps=eps) if post_layer_norm else None

    def forward(self, x):
        rows = x.reshape(-1, x.shape[-1])
        pre = self.i2h_proj(self.pre_layer_norm(rows))
        hid = offn.apply_activation(pre, "gelu_fused", self.gated)
        out = self.h2o_proj(hid)
        if self.post_layer_norm is not None:
            out = self.post_layer_norm(out)
        return (out + rows).view(x.shape)
