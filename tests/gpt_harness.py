"""A minimal causal language model around LeanFFN, in stock PyTorch, for the full-model parity case (test infrastructure).

It restates the parts of the reference's GPT that surround the feedforward block, so that every layer's FFN can be
switched between the HIP kernels (`lean_transformer_amd.LeanFFN`) and the plain-autograd oracle (`oracle.ffn.plain_ffn`)
with everything else identical:

  embeddings      word embedding [vocab, E] with a zeroed padding row, LayerNorm(E), Linear(E -> H) when E != H
                  (lean_transformer/models/gpt.py:89-147)
  layer x L       attention: pre-LN, fused qkv projection, rotary q/k, scores + additive causal mask of -10000,
                  softmax, value product, output projection, residual in fp32; the attention core is recomputed in
                  backward (lean_transformer/attn.py:66-149, lean_transformer/rotary.py:48-68)
                  then the FFN (lean_transformer/transformer.py:62-76)
  final LN        lean_transformer/transformer.py:33,84
  head            Linear(H -> E) initialised as the transpose of the embedding mapping + activation + LayerNorm(E) when
                  E != H, logits against the tied word embedding + a logits bias (lean_transformer/models/gpt.py:150-194)
  loss            next-token cross entropy, last position ignored (lean_transformer/models/gpt.py:286-293)
  init            N(0, initializer_range) weights with initializer_range = sqrt(2 / (5 H)), zero biases
                  (lean_transformer/config.py:113-116,210-228)
"""
import math
from dataclasses import dataclass
from typing import Optional

import torch
import torch.nn as nn
import torch.nn.functional as F
from torch.utils.checkpoint import checkpoint

from oracle import ffn as offn


@dataclass
class GPTConfig:
    vocab_size: int = 10000
    embedding_size: int = 1024
    hidden_size: int = 768
    num_layers: int = 12
    num_heads: int = 16
    intermediate_size: int = 3072
    gated: bool = True
    layer_norm_eps: float = 1e-12
    rotary_base: int = 10000
    pad_token_id: int = 0
    checkpoint_attention_core: bool = True

    @property
    def initializer_range(self) -> float:
        return math.sqrt(2.0 / (5.0 * self.hidden_size))


def rotary_tables(seq_len: int, dim: int, base: int, device):
    """cos / sin of position * base^(-2i/dim), the half-table repeated twice along the feature axis"""
    exponents = torch.linspace(0, -1 + 2 / dim, dim // 2, dtype=torch.float32, device=device)
    inv_freq = torch.pow(torch.tensor(float(base), device=device), exponents).repeat(2)
    angles = torch.arange(seq_len, dtype=torch.float32, device=device)[:, None] * inv_freq[None, :]
    return angles.cos(), angles.sin()


def apply_rotary(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """x [batch, seq, heads, dim]: (left, right) halves -> x * cos + (-right, left) * sin"""
    left, right = x.chunk(2, dim=-1)
    return x * cos[None, :, None, :] + torch.cat([-right, left], dim=-1) * sin[None, :, None, :]


def attention_core(query, key, value, mask, cos, sin, num_heads: int):
    batch, seq, hidden = query.shape
    head = hidden // num_heads
    q = apply_rotary(query.view(batch, seq, num_heads, head), cos, sin).permute(0, 2, 1, 3)
    k = apply_rotary(key.view(batch, seq, num_heads, head), cos, sin).permute(0, 2, 3, 1) / math.sqrt(head)
    v = value.view(batch, seq, num_heads, head).permute(0, 2, 1, 3)
    scores = torch.matmul(q, k) + mask
    out = torch.matmul(torch.softmax(scores, dim=-1), v)
    return out.transpose(2, 1).flatten(2)


class Attention(nn.Module):
    def __init__(self, cfg: GPTConfig, linear_impl: str = "torch"):
        """linear_impl: "torch" (nn.Linear) or "hip" (lean_transformer_amd.GeneralizedLinear on the HIP kernels, the layer
        the reference builds for its attention projections: lean_transformer/transformer.py:48-61, config.py:172-182)"""
        super().__init__()
        self.cfg = cfg
        self.pre_layer_norm = nn.LayerNorm(cfg.hidden_size, eps=cfg.layer_norm_eps)
        if linear_impl == "hip":
            import lean_transformer_amd as lt
            self.qkv_proj = lt.GeneralizedLinear(lt.GeneralizedMatrix(cfg.hidden_size, 3 * cfg.hidden_size), 0, True)
            self.out_proj = lt.GeneralizedLinear(lt.GeneralizedMatrix(cfg.hidden_size, cfg.hidden_size), 0, True)
        else:
            self.qkv_proj = nn.Linear(cfg.hidden_size, 3 * cfg.hidden_size)
            self.out_proj = nn.Linear(cfg.hidden_size, cfg.hidden_size)

    def forward(self, x, mask, cos, sin):
        qkv = self.qkv_proj(self.pre_layer_norm(x))
        q, k, v = qkv.split(self.cfg.hidden_size, dim=-1)
        if self.cfg.checkpoint_attention_core and torch.is_grad_enabled():
            core = checkpoint(attention_core, q, k, v, mask, cos, sin, self.cfg.num_heads, use_reentrant=False)
        else:
            core = attention_core(q, k, v, mask, cos, sin, self.cfg.num_heads)
        return self.out_proj(core) + x.to(torch.float32)


class OracleFFN(nn.Module):
    """the oracle's plain-autograd feedforward block behind the parameter names of LeanFFN (dense projections)"""

    def __init__(self, hidden: int, intermediate: int, gated: bool, eps: float):
        super().__init__()
        self.gated, self.eps = gated, eps
        self.lean = False  # True: the memory-lean autograd.Function of the oracle instead of the plain composition
        self.pre_layer_norm = nn.LayerNorm(hidden, eps=eps)
        self.i2h_proj = nn.Linear(hidden, intermediate * (2 if gated else 1))
        self.h2o_proj = nn.Linear(intermediate, hidden)

    def forward(self, x):
        if self.lean:
            # the reference's own schedule in stock ops (the oracle's LeanFFNFunction: saves x and the pre-activation,
            # closed-form backward, custom_fwd / custom_bwd like _LeanFFN, so under autocast every matmul of forward and
            # backward takes bf16 operands): a second stock-op implementation whose roundings fall elsewhere
            p = offn.FFNParams(
                self.pre_layer_norm.weight, self.pre_layer_norm.bias,
                offn.LinearParams(self.i2h_proj.weight, self.i2h_proj.bias, out_features=self.i2h_proj.out_features),
                offn.LinearParams(self.h2o_proj.weight, self.h2o_proj.bias, out_features=self.h2o_proj.out_features),
                None, None, offn.FFNConfig(gated=self.gated, act="gelu_fused", ln_eps=self.eps, residual=True, dropout=0.0))
            return offn.lean_ffn(x, p)
        autocast = torch.is_autocast_enabled(x.device.type)
        cast = (lambda t: t.to(torch.get_autocast_dtype(x.device.type))) if autocast else (lambda t: t)
        # under autocast the oracle follows the reference's roundings: LayerNorm in fp32, GEMM operands in bf16
        p = offn.FFNParams(
            self.pre_layer_norm.weight, self.pre_layer_norm.bias,
            offn.LinearParams(cast(self.i2h_proj.weight), cast(self.i2h_proj.bias), out_features=self.i2h_proj.out_features),
            offn.LinearParams(cast(self.h2o_proj.weight), cast(self.h2o_proj.bias), out_features=self.h2o_proj.out_features),
            None, None, offn.FFNConfig(gated=self.gated, act="gelu_fused", ln_eps=self.eps, residual=True, dropout=0.0))
        if not autocast:
            return offn.plain_ffn(x, p)
        with torch.autocast(x.device.type, enabled=False):
            return _oracle_ffn_bf16(x, p)


def _oracle_ffn_bf16(x: torch.Tensor, p: "offn.FFNParams") -> torch.Tensor:
    """plain_ffn with the mixed-precision roundings of the reference under autocast(bfloat16): fp32 LayerNorm, bf16 GEMM
    operands and pre-activation, fp32 residual stream (lean_transformer/ffn.py:184-207 with autocast's cast rules)"""
    shape = x.shape
    x2 = x.reshape(-1, shape[-1]).float()
    u = F.layer_norm(x2, x2.shape[-1:], p.ln_weight.float(), p.ln_bias.float(), p.cfg.ln_eps).to(torch.bfloat16)
    pre = F.linear(u, p.i2h.weight, p.i2h.bias)
    hid = offn.apply_activation(pre.float(), p.cfg.act, p.cfg.gated).to(torch.bfloat16)
    out = F.linear(hid, p.h2o.weight, p.h2o.bias)
    return (out.float() + x2).view(shape)


class MiniLeanGPT(nn.Module):
    def __init__(self, cfg: GPTConfig, ffn_impl: str, linear_impl: str = "torch"):
        """ffn_impl: "hip" (lean_transformer_amd.LeanFFN, GPU only) or "oracle" (stock PyTorch, any device);
        linear_impl: what the attention projections are, "torch" or "hip" (see Attention)"""
        super().__init__()
        self.cfg = cfg
        E, H = cfg.embedding_size, cfg.hidden_size
        self.word_embeddings = nn.Embedding(cfg.vocab_size, E, padding_idx=cfg.pad_token_id)
        self.embedding_layer_norm = nn.LayerNorm(E, eps=cfg.layer_norm_eps)
        self.embedding_hidden_mapping = nn.Linear(E, H) if E != H else None
        self.attentions = nn.ModuleList([Attention(cfg, linear_impl) for _ in range(cfg.num_layers)])
        if ffn_impl == "hip":
            import lean_transformer_amd as lt
            make = lambda: lt.LeanFFN(H, cfg.intermediate_size, gated=cfg.gated, layer_norm_eps=cfg.layer_norm_eps)
        elif ffn_impl == "oracle":
            make = lambda: OracleFFN(H, cfg.intermediate_size, cfg.gated, cfg.layer_norm_eps)
        else:
            raise ValueError(ffn_impl)
        self.ffns = nn.ModuleList([make() for _ in range(cfg.num_layers)])
        self.post_layer_norm = nn.LayerNorm(H, eps=cfg.layer_norm_eps)
        if E != H:
            self.head_bias = nn.Parameter(torch.zeros(E))
            self.head_mapping = nn.Parameter(torch.empty(E, H))
            self.head_layer_norm = nn.LayerNorm(E)
        self.logits_bias = nn.Parameter(torch.zeros(cfg.vocab_size))
        self.reset_parameters()

    @torch.no_grad()
    def reset_parameters(self, seed: int = 0):
        """every matrix ~ N(0, initializer_range) from a CPU generator in module order, biases 0, LayerNorm (1, 0)"""
        gen = torch.Generator().manual_seed(seed)
        std = self.cfg.initializer_range
        for module in self.modules():
            if isinstance(module, (nn.Linear, nn.Embedding)) or type(module).__name__ == "GeneralizedLinear":
                module.weight.copy_(torch.randn(module.weight.shape, generator=gen) * std)
                if getattr(module, "bias", None) is not None:
                    module.bias.zero_()
            elif isinstance(module, nn.LayerNorm):
                module.weight.fill_(1.0)
                module.bias.zero_()
        self.word_embeddings.weight[self.cfg.pad_token_id].zero_()
        if self.embedding_hidden_mapping is not None:
            self.head_mapping.copy_(self.embedding_hidden_mapping.weight.t())
            self.head_bias.zero_()
        self.logits_bias.zero_()

    def forward(self, input_ids: torch.Tensor, labels: Optional[torch.Tensor] = None):
        cfg = self.cfg
        batch, seq = input_ids.shape
        device = input_ids.device
        x = self.embedding_layer_norm(self.word_embeddings(input_ids))
        if self.embedding_hidden_mapping is not None:
            x = self.embedding_hidden_mapping(x)
        causal = torch.tril(torch.ones(seq, seq, dtype=torch.float32, device=device)).view(1, 1, seq, seq)
        mask = (1.0 - causal) * -10000.0
        cos, sin = rotary_tables(seq, cfg.hidden_size // cfg.num_heads, cfg.rotary_base, device)
        for attention, ffn in zip(self.attentions, self.ffns):
            x = attention(x, mask, cos, sin)
            x = ffn(x)
        x = self.post_layer_norm(x)
        if self.embedding_hidden_mapping is not None:
            x = F.linear(x, self.head_mapping, self.head_bias)
            x = self.head_layer_norm(offn.gelu_fused(x))
        logits = F.linear(x, self.word_embeddings.weight, self.logits_bias)
        if labels is None:
            return logits
        shifted = torch.cat([labels[:, 1:], torch.full_like(labels[:, :1], -100)], dim=1)
        loss = F.cross_entropy(logits.view(-1, logits.shape[-1]).float(), shifted.view(-1), ignore_index=-100)
        return loss, logits


def canonical_name(name: str) -> str:
    """parameter name with the generalized linear layer's `matrix.` level removed (qkv_proj.matrix.weight -> qkv_proj.weight)"""
    return name.replace(".matrix.weight", ".weight")


def copy_parameters(src: MiniLeanGPT, dst: MiniLeanGPT):
    """the implementations share parameter names up to the `matrix.` level of a generalized linear layer"""
    source = {canonical_name(k): v for k, v in src.state_dict().items()}
    with torch.no_grad():
        for name, tensor in dst.state_dict().items():
            tensor.copy_(source.pop(canonical_name(name)))
    assert not source, sorted(source)
