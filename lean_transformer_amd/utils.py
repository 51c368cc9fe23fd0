"""Activations for the FFN block.

``ACT2FN["gelu_fused"]`` (the default of LeanFFN) is the tanh-approximated GELU of the reference
(lean_transformer/utils.py:24-50, ACT2FN at utils.py:80).  Every callable defined here carries ``lt_act_kind``: the name
under which the HIP kernels evaluate it (and its derivative) in registers.  ``activation_kind`` maps a user-supplied callable
to such a name; a callable it does not recognise cannot run on the custom-gradient path.
"""
import torch
import torch.nn.functional as F

# kernel-side enumerators (keep in sync with include/leanffn.h: LT_ACT_*)
ACT_KINDS = {"gelu_fused": 0, "gelu": 1, "relu": 2, "silu": 3}


class GELU(torch.autograd.Function):
    """tanh-approximated GELU with a closed-form backward; reference: GELU, utils.py:41-50."""

    @staticmethod
    def forward(ctx, input: torch.Tensor):
        ctx.save_for_backward(input)
        return input * 0.5 * (1.0 + torch.tanh(0.79788456 * input * (1 + 0.044715 * input * input)))

    @staticmethod
    def backward(ctx, grad_output: torch.Tensor):
        (x,) = ctx.saved_tensors
        t = torch.tanh(0.79788456 * x * (1 + 0.044715 * x * x))
        jac = 0.5 * x * ((1 - t * t) * (0.79788456 + 0.1070322243 * x * x)) + 0.5 * (1 + t)
        return jac * grad_output


def _tag(fn, kind):
    fn.lt_act_kind = kind
    return fn


def gelu_fused(x):
    return GELU.apply(x)


def _gelu(x):
    return F.gelu(x)


def _relu(x):
    return F.relu(x)


def _silu(x):
    return F.silu(x)


_NATIVE = {
    "gelu_fused": _tag(gelu_fused, "gelu_fused"),
    "gelu_new": _tag(lambda x: F.gelu(x, approximate="tanh"), "gelu_fused"),
    "gelu_pytorch_tanh": _tag(lambda x: F.gelu(x, approximate="tanh"), "gelu_fused"),
    "gelu": _tag(_gelu, "gelu"),
    "relu": _tag(_relu, "relu"),
    "silu": _tag(_silu, "silu"),
    "swish": _tag(_silu, "silu"),
}


class _ActivationTable(dict):
    """The natively supported activations; any other name is looked up in Hugging Face's table when that is installed
    (such activations only work with ``ffn_custom_grad=False``)."""

    def __missing__(self, key):
        try:
            from transformers.activations import ACT2FN as HF_ACT2FN
        except ImportError:  # pragma: no cover
            raise KeyError(key)
        return HF_ACT2FN[key]


ACT2FN = _ActivationTable(_NATIVE)


def activation_kind(activation) -> str:
    """Name of the kernel-side activation that equals ``activation``, or raise NotImplementedError."""
    kind = getattr(activation, "lt_act_kind", None)
    if kind is not None:
        return kind
    if activation is GELU.apply:
        return "gelu_fused"
    if activation in (F.gelu, torch.nn.functional.gelu):
        return "gelu"
    if activation in (F.relu, torch.relu):
        return "relu"
    if activation is F.silu:
        return "silu"
    if isinstance(activation, torch.nn.GELU):
        return "gelu_fused" if activation.approximate == "tanh" else "gelu"
    if isinstance(activation, torch.nn.ReLU):
        return "relu"
    if isinstance(activation, torch.nn.SiLU):
        return "silu"
    name = type(activation).__name__
    by_class = {"GELUActivation": "gelu", "NewGELUActivation": "gelu_fused", "PytorchGELUTanh": "gelu_fused",
                "GELUTanh": "gelu_fused", "FastGELUActivation": "gelu_fused", "SiLUActivation": "silu"}
    if name in by_class:
        return by_class[name]
    raise NotImplementedError(
        f"activation {activation!r} has no HIP implementation (supported: {sorted(ACT_KINDS)}); "
        "construct LeanFFN with ffn_custom_grad=False to run it through stock PyTorch ops")
