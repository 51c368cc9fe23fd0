"""Activations for the FFN block.

``ACT2FN["gelu_fused"]`` (the default of LeanFFN) is the tanh-approximated GELU of the reference
(lean_transformer/utils.py:24-50, ACT2FN at utils.py:80).  Every callable defined here carries ``lt_act_kind``: the name
under which the HIP kernels evaluate it (and its derivative) in registers.  ``activation_kind`` maps a user-supplied callable
to such a name; a callable it does not recognise cannot run on the custom-gradient path.
"""
import torch
import torch.nn.functional as F

# kernel-side enumerators (keep in sync with include/leanffn.h: LT_ACT_*)
ACT_KINDS = {"gelu_fused": 0, "gelu": 1, "relu": 2, "silu": 3, "quick_gelu": 4, "gelu_10": 5, "relu6": 6, "relu2": 7,
             "leaky_relu": 8, "mish": 9, "sigmoid": 10, "tanh": 11, "linear": 12, "hardswish": 13, "laplace": 14,
             "sqrtsoftplus": 15}


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


def _laplace(x, mu=0.707107, sigma=0.282095):
    return 0.5 * (1.0 + torch.erf((x - mu) / (sigma * 2.0 ** 0.5)))


# name -> (stock-op callable, kernel-side kind).  The names are those of transformers.activations.ACT2FN, the table the
# reference extends (utils.py:80); the tanh-form GELUs of that table differ from gelu_fused only in digits of sqrt(2 / pi)
# beyond fp32 resolution and share its kernel.  Entries with learned parameters (prelu, xielu) are not here: they resolve to
# Hugging Face's modules and run with ffn_custom_grad=False only.
_NATIVE = {name: _tag(fn, kind) for name, fn, kind in (
    ("gelu_fused", gelu_fused, "gelu_fused"),
    ("gelu_new", lambda x: F.gelu(x, approximate="tanh"), "gelu_fused"),
    ("gelu_pytorch_tanh", lambda x: F.gelu(x, approximate="tanh"), "gelu_fused"),
    ("gelu_python_tanh", lambda x: F.gelu(x, approximate="tanh"), "gelu_fused"),
    ("gelu_fast", lambda x: F.gelu(x, approximate="tanh"), "gelu_fused"),
    ("gelu_accurate", lambda x: F.gelu(x, approximate="tanh"), "gelu_fused"),
    ("gelu", lambda x: F.gelu(x), "gelu"),
    ("gelu_python", lambda x: F.gelu(x), "gelu"),
    ("relu", lambda x: F.relu(x), "relu"),
    ("silu", lambda x: F.silu(x), "silu"),
    ("swish", lambda x: F.silu(x), "silu"),
    ("quick_gelu", lambda x: x * torch.sigmoid(1.702 * x), "quick_gelu"),
    ("gelu_10", lambda x: torch.clip(F.gelu(x), -10, 10), "gelu_10"),
    ("relu6", lambda x: F.relu6(x), "relu6"),
    ("relu2", lambda x: torch.square(F.relu(x)), "relu2"),
    ("leaky_relu", lambda x: F.leaky_relu(x, 0.01), "leaky_relu"),
    ("mish", lambda x: F.mish(x), "mish"),
    ("sigmoid", lambda x: torch.sigmoid(x), "sigmoid"),
    ("tanh", lambda x: torch.tanh(x), "tanh"),
    ("linear", lambda x: x, "linear"),
    ("hardswish", lambda x: F.hardswish(x), "hardswish"),
    ("laplace", _laplace, "laplace"),
    ("sqrtsoftplus", lambda x: F.softplus(x).sqrt(), "sqrtsoftplus"),
)}


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


# callables and module classes that name a kernel-side activation without carrying the tag
_BY_FUNCTION = {F.gelu: "gelu", F.relu: "relu", torch.relu: "relu", F.silu: "silu", F.relu6: "relu6", F.mish: "mish",
                torch.sigmoid: "sigmoid", F.sigmoid: "sigmoid", torch.tanh: "tanh", F.tanh: "tanh", F.hardswish: "hardswish"}
_BY_CLASS = {  # torch.nn modules and the classes of transformers.activations (matched by name: no import needed)
    "ReLU": "relu", "SiLU": "silu", "ReLU6": "relu6", "Mish": "mish", "Sigmoid": "sigmoid", "Tanh": "tanh",
    "Hardswish": "hardswish", "Identity": "linear",
    "GELUActivation": "gelu", "NewGELUActivation": "gelu_fused", "PytorchGELUTanh": "gelu_fused", "GELUTanh": "gelu_fused",
    "FastGELUActivation": "gelu_fused", "AccurateGELUActivation": "gelu_fused", "SiLUActivation": "silu",
    "QuickGELUActivation": "quick_gelu", "ReLUSquaredActivation": "relu2", "MishActivation": "mish",
    "LinearActivation": "linear", "LaplaceActivation": "laplace", "SqrtSoftplusActivation": "sqrtsoftplus",
}


def activation_kind(activation) -> str:
    """Name of the kernel-side activation that equals ``activation``, or raise NotImplementedError."""
    kind = getattr(activation, "lt_act_kind", None)
    if kind is not None:
        return kind
    if activation is GELU.apply:
        return "gelu_fused"
    try:
        if activation in _BY_FUNCTION:
            return _BY_FUNCTION[activation]
    except TypeError:  # unhashable callable
        pass
    name = type(activation).__name__
    if isinstance(activation, torch.nn.GELU):
        return "gelu_fused" if activation.approximate == "tanh" else "gelu"
    if isinstance(activation, torch.nn.LeakyReLU) and activation.negative_slope == 0.01:
        return "leaky_relu"
    if name == "ClippedGELUActivation" and (activation.min, activation.max) == (-10, 10):
        return "gelu_10"
    if name in _BY_CLASS and not any(True for _ in getattr(activation, "parameters", lambda: ())()):
        return _BY_CLASS[name]
    raise NotImplementedError(
        f"activation {activation!r} has no HIP implementation (supported: {sorted(ACT_KINDS)}); "
        "construct LeanFFN with ffn_custom_grad=False to run it through stock PyTorch ops")
