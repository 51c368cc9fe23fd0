"""Weight containers and the "generalized linear" layer: (dense | block-sparse) main matrix + optional low-rank term,
shareable between layers, with a per-layer low-rank adapter.

Same classes, constructor arguments, attributes and state_dict keys as lean_transformer/blocksparse/linear.py:19-149, so a
checkpoint of the reference loads unchanged.  The forward / backward of ``_GeneralizedLinear`` run on the HIP kernels
(lt_linear_forward / lt_linear_backward) instead of F.linear / addmm / the embedding_bag-based sparse matmul.
"""
import math
from typing import Optional, Tuple

import torch
import torch.nn as nn

from .. import _native as nat
from .layout import get_blocksparse_layout, get_indices_from_layout


def _small_init_std(in_features: int, out_features: int) -> float:
    """standard deviation the sparse blocks and the shared low-rank factors start from: sqrt(2 / (5 min(fan)))"""
    return math.sqrt(0.4 / min(in_features, out_features))


class GeneralizedMatrix(nn.Module):
    """Weights of one linear map, held apart from the layers that apply it so that several layers can share them.

    ``weight`` is either a dense ``[out_features, in_features]`` matrix (``blocksparse_layout=None``) or the active blocks
    of a block-sparse one in the "native" order ``[in_features, active blocks per input block, block]`` together with three
    persistent buffers: the boolean block ``layout`` and the ``forward_indices`` / ``backward_indices`` tables built from
    it.  ``lowrank_dim > 0`` adds the factors ``lowrank_first [r, in]`` and ``lowrank_second [out, r]`` of an additive
    low-rank term.  Names and shapes are those of lean_transformer/blocksparse/linear.py:19-66.
    """

    def __init__(self, in_features: int, out_features: int, blocksparse_layout: Optional[str] = None,
                 lowrank_dim: int = 0, blocksparse_backend: str = 'native'):
        super().__init__()
        if blocksparse_backend != 'native':
            raise NotImplementedError(
                f"blocksparse_backend={blocksparse_backend!r}: only the 'native' weight format is implemented "
                "(its matmul runs on HIP kernels; there is no Triton path)")
        self.in_features, self.out_features = in_features, out_features
        self.blocksparse_backend = blocksparse_backend
        std = _small_init_std(in_features, out_features)

        if blocksparse_layout is not None:
            layout = get_blocksparse_layout(out_features, in_features, blocksparse_layout)
            out_blocks, in_blocks = layout.shape
            if in_features % in_blocks or out_features % out_blocks or in_features // in_blocks != out_features // out_blocks:
                raise AssertionError(f"layout {tuple(layout.shape)} does not cut a {out_features} x {in_features} matrix "
                                     "into square blocks")
            block = in_features // in_blocks
            forward_indices, backward_indices = get_indices_from_layout(layout)
            for name, table in (("layout", layout), ("forward_indices", forward_indices),
                                ("backward_indices", backward_indices)):
                self.register_buffer(name, table, persistent=True)
            blocks_per_input = forward_indices.numel() // in_blocks
            self.weight = nn.Parameter(torch.empty(in_features, blocks_per_input, block).normal_(std=std))
        else:
            self.layout = self.forward_indices = self.backward_indices = None
            self.weight = nn.Parameter(torch.empty(out_features, in_features))
            nn.init.kaiming_uniform_(self.weight, a=math.sqrt(5))  # what nn.Linear does

        self.lowrank_first = self.lowrank_second = None
        if lowrank_dim:
            self.lowrank_first = nn.Parameter(torch.empty(lowrank_dim, in_features).normal_(std=std))
            self.lowrank_second = nn.Parameter(torch.empty(out_features, lowrank_dim).normal_(std=std))

    @property
    def shape(self):
        return self.out_features, self.in_features

    @property
    def matmul_op(self):
        """The reference's slot for a Triton matmul object; always None here (the 'native' format is the only one)."""
        return None

    def __repr__(self):
        return f"{type(self).__name__}({self.out_features}, {self.in_features})"

    def forward(self, input: torch.Tensor, *, ignore_lowrank: bool = False):
        """``input @ W^T`` like a bias-free ``nn.Linear``; the low-rank term is added unless ``ignore_lowrank``"""
        first, second = (None, None) if ignore_lowrank else (self.lowrank_first, self.lowrank_second)
        return _GeneralizedLinear.apply(input, self.weight, None, first, second, self.forward_indices,
                                        self.backward_indices, None)


class GeneralizedLinear(nn.Linear):
    """``nn.Linear`` look-alike over a (possibly shared) ``GeneralizedMatrix``, with its own bias and an optional low-rank
    adapter ``adapter_first [a, in]``, ``adapter_second [out, a]`` that belongs to this layer alone
    (lean_transformer/blocksparse/linear.py:106-149)."""

    def __init__(self, matrix: GeneralizedMatrix, adapter_dim: int = 0, bias: bool = True):
        nn.Module.__init__(self)  # not nn.Linear.__init__: that would allocate a weight of its own
        self.matrix = matrix
        self.out_features, self.in_features = matrix.shape
        self.bias = nn.Parameter(torch.zeros(self.out_features)) if bias else None
        self.adapter_first = self.adapter_second = None
        if adapter_dim:
            # LoRA-style start (arXiv:2106.09685): random input factor, zero output factor, so the adapter begins as a no-op
            self.adapter_first = nn.Parameter(nn.init.xavier_normal_(torch.empty(adapter_dim, self.in_features)))
            self.adapter_second = nn.Parameter(torch.zeros(self.out_features, adapter_dim))

    def get_combined_lowrank_components(self) -> Tuple[Optional[torch.Tensor], Optional[torch.Tensor]]:
        """One (first [r + a, in], second [out, r + a]) pair covering the matrix's shared low-rank term and this layer's
        adapter, so that both ride in a single pair of skinny GEMMs; (None, None) when the layer has neither."""
        firsts = [t for t in (self.matrix.lowrank_first, self.adapter_first) if t is not None]
        seconds = [t for t in (self.matrix.lowrank_second, self.adapter_second) if t is not None]
        if not firsts:
            return None, None
        if len(firsts) == 1:
            return firsts[0], seconds[0]
        return torch.cat(firsts, dim=0), torch.cat(seconds, dim=1)

    @property
    def weight(self):
        return self.matrix.weight

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        first, second = self.get_combined_lowrank_components()
        return _GeneralizedLinear.apply(input, self.weight, self.bias, first, second, self.matrix.forward_indices,
                                        self.matrix.backward_indices, self.matrix.matmul_op)


def compute_dtype_for(weight: torch.Tensor) -> torch.dtype:
    """dtype of GEMM operands: the autocast dtype when autocast is on (as F.linear would use), else the weight's dtype"""
    if torch.is_autocast_enabled("cuda"):
        dtype = torch.get_autocast_dtype("cuda")
        if dtype not in (torch.bfloat16, torch.float16):
            raise NotImplementedError(f"autocast to {dtype}: the HIP kernels compute in bfloat16, float16 or float32")
        return dtype
    return weight.dtype


def _as(t: Optional[torch.Tensor], dtype: torch.dtype) -> Optional[torch.Tensor]:
    if t is None:
        return None
    t = t.detach()
    if t.dtype != dtype:
        t = t.to(dtype)
    return t.contiguous()


def shared_list_run(forward_indices: torch.Tensor, blocks_per_in: int) -> int:
    """Largest power of two g such that every aligned run of g consecutive output blocks has the same list of input blocks
    (1 when neighbouring output blocks differ).  PixelFly with ``stretch=True`` on a matrix with more output than input
    blocks repeats every list ``out_blocks / in_blocks`` times; the weight-gradient kernel reads dY once per run of 4
    instead of once per output block when told so.  Computed once per index tensor (one device -> host sync) and remembered
    on the tensor object itself together with the tensor's version counter, so an in-place change recomputes it."""
    cached = getattr(forward_indices, "_lt_shared_list_run", None)
    if cached is not None and cached[0] == (forward_indices._version, blocks_per_in):
        return cached[1]
    lists = torch.div(forward_indices, blocks_per_in, rounding_mode="floor")  # input block of every entry
    run, n_out = 1, lists.shape[0]
    while n_out % (2 * run) == 0:
        grouped = lists.reshape(n_out // (2 * run), 2 * run, -1)
        # ... and the run's weight blocks must sit next to each other under every input block of the list (they do when the
        # index tables list active blocks in ascending order, as get_indices_from_layout builds them): the kernels read them
        # as one matrix
        flat = forward_indices.reshape(n_out // (2 * run), 2 * run, -1)
        step = torch.arange(2 * run, device=flat.device, dtype=flat.dtype)[None, :, None]
        if not bool(((grouped == grouped[:, :1]) & (flat == flat[:, :1] + step)).all()):
            break
        run *= 2
    forward_indices._lt_shared_list_run = ((forward_indices._version, blocks_per_in), run)
    return run


def _strided_run(lists: torch.Tensor) -> Tuple[int, int]:
    """(g, s): the most members g (a power of two, g * s = number of blocks) such that blocks r, r + s, r + 2 s, ... all have the
    same row in `lists` -- what tiling a square pattern s blocks wide g times gives; (1, 1) when there is no such structure"""
    n = lists.shape[0]
    g = 1
    while n % (2 * g) == 0:
        g *= 2
    while g >= 2:
        tiled = lists.reshape(g, n // g, -1)
        if bool((tiled == tiled[:1]).all()):
            return g, n // g
        g //= 2
    return 1, 1


def shared_list_group(forward_indices: torch.Tensor, blocks_per_in: int) -> int:
    """lt_linear.out_group of a layer with these index tables: the run of consecutive output blocks with one list of input
    blocks (shared_list_run) when that is 4 or more; else, when output blocks a fixed number of blocks apart share their lists
    (PixelFly with ``stretch=False`` on a tall matrix tiles the square butterfly), the number of such blocks in the low 16
    bits and their distance in the high 16 bits; else the run (1 ... 2).  Remembered on the tensor like shared_list_run."""
    run = shared_list_run(forward_indices, blocks_per_in)
    if run >= 4:
        return run
    cached = getattr(forward_indices, "_lt_shared_list_group", None)
    if cached is not None and cached[0] == (forward_indices._version, blocks_per_in):
        return cached[1]
    members, stride = _strided_run(torch.div(forward_indices, blocks_per_in, rounding_mode="floor"))
    group = (members | (stride << 16)) if (members >= 4 and 1 < stride < 1 << 15 and members < 1 << 16) else run
    forward_indices._lt_shared_list_group = ((forward_indices._version, blocks_per_in), group)
    return group


def shared_input_group(backward_indices: torch.Tensor) -> int:
    """lt_linear.in_group: the same on the input side (shared_input_run, else blocks a fixed distance apart)"""
    run = shared_input_run(backward_indices)
    if run >= 4:
        return run
    cached = getattr(backward_indices, "_lt_shared_input_group", None)
    if cached is not None and cached[0] == backward_indices._version:
        return cached[1]
    members, stride = _strided_run(backward_indices)
    group = (members | (stride << 16)) if (members >= 4 and 1 < stride < 1 << 15 and members < 1 << 16) else run
    backward_indices._lt_shared_input_group = (backward_indices._version, group)
    return group


def shared_input_run(backward_indices: torch.Tensor) -> int:
    """The same on the input side: the largest power of two g such that every aligned run of g consecutive input blocks has
    the same list of output blocks (PixelFly with ``stretch=True`` on a matrix with more input than output blocks: ``in_blocks
    / out_blocks``).  Remembered on the tensor like shared_list_run."""
    cached = getattr(backward_indices, "_lt_shared_input_run", None)
    if cached is not None and cached[0] == backward_indices._version:
        return cached[1]
    run, n_in = 1, backward_indices.shape[0]
    while n_in % (2 * run) == 0:
        grouped = backward_indices.reshape(n_in // (2 * run), 2 * run, -1)
        if not bool((grouped == grouped[:, :1]).all()):
            break
        run *= 2
    backward_indices._lt_shared_input_run = (backward_indices._version, run)
    return run


def linear_desc(weight, bias_f32, lowrank_first, lowrank_second, forward_indices, backward_indices,
                index_owner: Optional[torch.Tensor] = None, backward_owner: Optional[torch.Tensor] = None) -> "nat.LtLinear":
    """ctypes descriptor of one projection; all tensors already in their final dtype and contiguous.  index_owner /
    backward_owner: the caller's own forward_indices / backward_indices tensors (the module's buffers) when the ones passed
    may be converted copies of them: the shared-list runs are remembered on those objects, so that a copy made per call
    does not recompute them (and synchronise) per call."""
    desc = nat.LtLinear()
    desc.weight = nat.ptr(weight)
    desc.bias = nat.ptr(bias_f32)
    desc.lowrank_first, desc.lowrank_second = nat.ptr(lowrank_first), nat.ptr(lowrank_second)
    desc.lowrank = 0 if lowrank_first is None else lowrank_first.shape[0]
    if forward_indices is None:
        desc.out_features, desc.in_features = weight.shape
        desc.block = desc.blocks_per_in = desc.blocks_per_out = 0
    else:
        in_features, blocks_per_in, block = weight.shape
        desc.in_features, desc.out_features = in_features, forward_indices.shape[0] * block
        desc.block, desc.blocks_per_in, desc.blocks_per_out = block, blocks_per_in, forward_indices.shape[1]
        desc.forward_indices, desc.backward_indices = nat.ptr(forward_indices), nat.ptr(backward_indices)
        owner = forward_indices if index_owner is None else index_owner
        desc.out_group = shared_list_group(owner, blocks_per_in)
        if backward_indices is not None:
            desc.in_group = shared_input_group(backward_indices if backward_owner is None else backward_owner)
    return desc


class _GeneralizedLinear(torch.autograd.Function):
    """y = x W^T (+ bias) (+ (x L1^T) L2^T) with W dense or block-sparse.  Argument order as in the reference's
    _GeneralizedLinear.apply (linear.py:147-149): input, main_weight, bias, lowrank_first, lowrank_second,
    forward_indices, backward_indices[, matmul_op]."""

    @staticmethod
    def forward(ctx, *args):
        ctx._nargs = len(args)
        (input, main_weight, bias, lowrank_first, lowrank_second, forward_indices, backward_indices,
         matmul_op) = tuple(args) + (None,) * (8 - len(args))
        if matmul_op is not None:
            raise NotImplementedError("matmul_op plug-ins (Triton) are not supported; the block-sparse matmul is built in")
        device = nat.require_gpu(input, main_weight, bias, lowrank_first, lowrank_second, forward_indices, backward_indices)
        dtype = compute_dtype_for(main_weight)
        x = _as(input, dtype).reshape(-1, input.shape[-1])
        w = _as(main_weight, dtype)
        l1, l2 = _as(lowrank_first, dtype), _as(lowrank_second, dtype)
        b32 = _as(bias, torch.float32)
        fwd = None if forward_indices is None else forward_indices.to(torch.int32).contiguous()
        bwd = None if backward_indices is None else backward_indices.to(torch.int64).contiguous()
        desc = linear_desc(w, b32, l1, l2, fwd, bwd, forward_indices, backward_indices)
        if x.shape[1] != desc.in_features:
            raise ValueError(f"input has {x.shape[1]} features, the weight takes {desc.in_features}")
        tokens = x.shape[0]
        y = torch.empty(tokens, desc.out_features, dtype=dtype, device=device)
        hid = torch.empty(tokens, desc.lowrank, dtype=dtype, device=device) if desc.lowrank else None
        if tokens > 0:
            lib = nat.lib(dtype)
            nat.check(lib.lt_linear_forward(desc, tokens, nat.dtype_code(dtype), nat.ptr(x), nat.ptr(y), nat.ptr(hid),
                                            nat.current_stream(device)), "lt_linear_forward", lib)
        ctx.save_for_backward(input, hid, main_weight, lowrank_first, lowrank_second, forward_indices, backward_indices)
        ctx._dtype, ctx._has_bias = dtype, bias is not None
        return y.view(*input.shape[:-1], desc.out_features)

    @staticmethod
    def backward(ctx, grad_output):
        input, hid, main_weight, lowrank_first, lowrank_second, forward_indices, backward_indices = ctx.saved_tensors
        dtype = ctx._dtype
        device = grad_output.device
        need = tuple(ctx.needs_input_grad) + (False,) * 8
        x = _as(input, dtype).reshape(-1, input.shape[-1])
        dy = _as(grad_output, dtype).reshape(x.shape[0], -1)
        w = _as(main_weight, dtype)
        l1, l2 = _as(lowrank_first, dtype), _as(lowrank_second, dtype)
        fwd = None if forward_indices is None else forward_indices.to(torch.int32).contiguous()
        bwd = None if backward_indices is None else backward_indices.to(torch.int64).contiguous()
        desc = linear_desc(w, None, l1, l2, fwd, bwd, forward_indices, backward_indices)
        tokens = x.shape[0]
        grads = nat.LtLinearGrads()
        dx = torch.empty_like(x) if need[0] else None
        dw = torch.empty_like(w) if need[1] else None
        db = torch.empty(desc.out_features, dtype=torch.float32, device=device) if (ctx._has_bias and need[2]) else None
        dl1 = torch.empty_like(l1) if (l1 is not None and need[3]) else None
        dl2 = torch.empty_like(l2) if (l2 is not None and need[4]) else None
        grads.weight, grads.bias, grads.lowrank_first, grads.lowrank_second = (nat.ptr(dw), nat.ptr(db), nat.ptr(dl1),
                                                                               nat.ptr(dl2))
        if tokens > 0:
            lib = nat.lib(dtype)
            ws = nat.workspace(lib.lt_linear_backward_workspace_bytes(desc, tokens, nat.dtype_code(dtype)), device)
            nat.check(lib.lt_linear_backward(desc, tokens, nat.dtype_code(dtype), nat.ptr(x), nat.ptr(dy), nat.ptr(hid),
                                             nat.ptr(dx), grads, nat.ptr(ws), ws.numel(), nat.current_stream(device)),
                      "lt_linear_backward", lib)
        else:
            for g in (dw, db, dl1, dl2):
                if g is not None:
                    g.zero_()
        out = (None if dx is None else dx.view(input.shape), dw, db, dl1, dl2, None, None, None)
        return out[:ctx._nargs]  # callers pass 2..8 positional arguments (everything after main_weight is optional)
