"""bf16 LeanFFN on the tiled MFMA kernels through every module knob that changes which epilogue strip or which k-segment
layout a launch takes: activations other than the tanh GELU, no residual, post-LayerNorm, dropout under activation
checkpointing, a bf16 residual stream at benchmark size, and dense projections with a low-rank term / adapter (a second
k-segment in the copy-based kernel, the skinny 128 x 128 tile for the rank factors).  All against the fp32 CPU oracle at the
bf16 bars (max relative error 2e-2, cosine 0.9999)."""
import pytest
import torch
from torch.utils.checkpoint import checkpoint

import lean_transformer_amd as lt
from conftest import assert_close
from helpers import dropout_mask, generator_position, module_tensors, oracle_params, run_oracle
from lean_transformer_amd.utils import ACT2FN
from test_gpu_ffn import _compare, _headline, _full_size_checks, _oracle_named_grads, _run_module

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
BF16 = torch.bfloat16


def _randomise_small_vectors(ffn, seed=0):
    g = torch.Generator().manual_seed(seed)
    with torch.no_grad():
        norms = [ffn.pre_layer_norm] + ([ffn.post_layer_norm] if ffn.post_layer_norm is not None else [])
        for ln in norms:
            ln.weight.copy_(torch.rand(ln.weight.shape, generator=g) + 0.5)
            ln.bias.copy_(torch.randn(ln.bias.shape, generator=g) * 0.2)
        for proj in (ffn.i2h_proj, ffn.h2o_proj):
            if proj.bias is not None:
                proj.bias.copy_(torch.randn(proj.bias.shape, generator=g) * 0.1)


KINKED = ("relu", "relu6", "leaky_relu", "hardswish")  # derivative jumps: see the docstring below
OTHER_ACTS = [(a, g, t) for a in ("gelu", "relu", "silu") for g in (False, True) for t in (512, 300)] + [
    (a, i % 2 == 0, 300 if i % 3 == 0 else 512) for i, a in enumerate(
        ("quick_gelu", "gelu_10", "relu6", "relu2", "leaky_relu", "mish", "sigmoid", "tanh", "linear", "hardswish", "laplace",
         "sqrtsoftplus", "gelu_accurate", "gelu_fast"))]


@pytest.mark.parametrize("act,gated,tokens", OTHER_ACTS)
def test_bf16_other_activations_take_the_general_epilogue_strips(act, gated, tokens):
    """the straight-line strips are compiled for the tanh GELU; every other activation goes through the strips that choose
    per row (forward activation epilogue, backward d-activation epilogue with its fused column sums).  Every closed-form
    entry of the Hugging Face table has a row.  The derivative of relu (and of relu6, leaky_relu, hardswish)
    jumps at 0, so its gradients depend on the sign of the pre-activation as stored (bf16): the oracle is asked to round
    where the bf16 path stores (LayerNorm output, pre-activation, activation output), which is what the reference does
    under bf16 autocast; the smooth activations are compared with the unrounded fp32 oracle like everywhere else."""
    torch.manual_seed(17)
    ffn = lt.LeanFFN(512, 1024, activation=ACT2FN[act], gated=gated, layer_norm_eps=1e-5)
    _randomise_small_vectors(ffn)
    ffn = ffn.to(DEV).to(BF16)
    _compare(ffn, torch.randn(tokens, 512), torch.randn(tokens, 512), BF16, bf16_rounding=(act in KINKED))


@pytest.mark.parametrize("io_dtype", [torch.float32, BF16])
@pytest.mark.parametrize("dropout", [0.0, 0.1])
def test_bf16_without_residual(io_dtype, dropout):
    """residual=False (reversible stacks add the input themselves): the down-projection epilogue has nothing to read"""
    torch.manual_seed(19)
    tokens, hidden = 512, 512
    ffn = lt.LeanFFN(hidden, 1024, gated=True, residual=False, dropout=dropout, layer_norm_eps=1e-5)
    _randomise_small_vectors(ffn)
    ffn = ffn.to(DEV).to(BF16)
    x, dy = torch.randn(tokens, hidden).to(io_dtype), torch.randn(tokens, hidden).to(io_dtype)
    torch.cuda.manual_seed(5)
    seed, offset = generator_position(DEV)
    mask = dropout_mask(tokens, hidden, dropout, seed, offset, torch.device(DEV)).cpu() if dropout else None
    _compare(ffn, x, dy, BF16, mask=mask)


@pytest.mark.parametrize("hidden,inter", [(512, 1024), (1024, 2048)])
@pytest.mark.parametrize("gated", [False, True])
@pytest.mark.parametrize("dropout", [0.0, 0.1])
def test_bf16_post_layer_norm(hidden, inter, gated, dropout):
    torch.manual_seed(23)
    tokens = 384
    ffn = lt.LeanFFN(hidden, inter, gated=gated, post_layer_norm=True, dropout=dropout, layer_norm_eps=1e-5)
    _randomise_small_vectors(ffn)
    ffn = ffn.to(DEV).to(BF16)
    x, dy = torch.randn(tokens, hidden), torch.randn(tokens, hidden)
    torch.cuda.manual_seed(6)
    seed, offset = generator_position(DEV)
    mask = dropout_mask(tokens, hidden, dropout, seed, offset, torch.device(DEV)).cpu() if dropout else None
    _compare(ffn, x, dy, BF16, mask=mask)


@pytest.mark.parametrize("dtype", [torch.float32, BF16])
def test_dropout_replays_under_activation_checkpointing(dtype):
    """torch.utils.checkpoint runs the forward twice (the second time inside backward, with the RNG state of the first
    restored): both must draw the same Philox sub-stream, i.e. the result must equal the un-checkpointed run of one seed"""
    torch.manual_seed(29)
    tokens, hidden = 512, 512
    ffn = lt.LeanFFN(hidden, 1024, gated=True, dropout=0.1, layer_norm_eps=1e-5)
    _randomise_small_vectors(ffn)
    ffn = ffn.to(DEV).to(dtype)
    x, dy = torch.randn(tokens, hidden), torch.randn(tokens, hidden)
    params = module_tensors(ffn)

    def run(use_checkpoint):
        torch.cuda.manual_seed(123)
        xd = x.to(DEV).requires_grad_(True)
        y = checkpoint(ffn, xd, use_reentrant=False) if use_checkpoint else ffn(xd)
        return y.detach(), torch.autograd.grad(y, [xd, *params], dy.to(DEV))

    y0, g0 = run(False)
    y1, g1 = run(True)
    assert torch.equal(y0, y1)
    for a, b in zip(g0, g1):
        assert torch.equal(a, b)
    torch.cuda.manual_seed(123)
    seed, offset = generator_position(DEV)
    mask = dropout_mask(tokens, hidden, 0.1, seed, offset, torch.device(DEV)).cpu()
    y_ref, dx_ref, g_ref = run_oracle(oracle_params(ffn), x, dy, mask)
    assert_close(y1, y_ref, dtype, "y")
    assert_close(g1[0], dx_ref, dtype, "dx")
    for i, (a, b) in enumerate(zip(g1[1:], g_ref)):
        assert_close(a, b, dtype, f"param grad {i}")


def test_custom_grad_switch_draws_the_same_dropout_mask():
    """reference tests/test_modifications.py:12-34: with dropout on, flipping ffn_custom_grad under one seed changes
    neither the output nor any gradient -- both paths must drop the same elements"""
    torch.manual_seed(31)
    ffn = lt.LeanFFN(256, 512, gated=True, dropout=0.1, post_layer_norm=True, layer_norm_eps=1e-5)
    _randomise_small_vectors(ffn)
    ffn = ffn.to(DEV)
    x = torch.randn(3, 70, 256, device=DEV)
    dy = torch.randn(3, 70, 256, device=DEV)
    results = []
    for custom in (True, False, True):
        ffn.ffn_custom_grad = custom
        torch.cuda.manual_seed(1337)
        xd = x.clone().requires_grad_(True)
        out = ffn(ffn(xd))  # two applications: the second draws the next sub-stream in both modes
        grads = torch.autograd.grad(out, [xd, *ffn.parameters()], dy)
        results.append((out.detach(), grads, generator_position(DEV)[1]))
    assert results[0][2] == results[1][2] == results[2][2]  # the generator advanced by the same amount
    assert torch.equal(results[0][0], results[2][0])
    assert_close(results[1][0], results[0][0], torch.float32, "output across the switch")
    for a, b in zip(results[1][1], results[0][1]):
        assert_close(a, b, torch.float32, "gradient across the switch")
    # without post-LN a dropped element of the output is exactly the residual: the two paths drop the same positions
    plain = lt.LeanFFN(256, 512, dropout=0.5, layer_norm_eps=1e-5).to(DEV)
    masks = []
    for custom in (True, False):
        plain.ffn_custom_grad = custom
        torch.cuda.manual_seed(7)
        masks.append(plain(x) == x)
    assert torch.equal(masks[0], masks[1]) and 0.4 < masks[0].float().mean().item() < 0.6


def test_config2_shape_bf16_residual_stream():
    """benchmark config 2's shape with x, y, dy, dx in bf16 as well (io_dtype = bf16): dropout 0.1, plain GELU"""
    ffn, x, dy = _headline(2048, 8192, False, 0.02, 0.1, (4, 2048))
    _full_size_checks(ffn, x.to(BF16), dy.to(BF16), 0.1)


@pytest.mark.parametrize("tokens", [1, 64, 300, 1024])
@pytest.mark.parametrize("gated", [False, True])
@pytest.mark.parametrize("lowrank_dim,adapter_dim", [(64, 0), (128, 0), (64, 64), (0, 128)])
def test_bf16_dense_projections_with_lowrank_and_adapter(tokens, gated, lowrank_dim, adapter_dim):
    """dense GeneralizedLinear projections with a shared low-rank term and / or a per-layer adapter, in bf16: the low-rank
    product rides as a second k-segment of the projection's launch, the rank factors run on the 128 x 128 tile with a split
    reduction, and with few tokens the fused column sums of the d-activation epilogue must stay inside their buffer (the
    workspace regions behind it hold the low-rank hidden gradient that the same launch reads)"""
    torch.manual_seed(tokens + lowrank_dim + 3 * adapter_dim + gated)
    hidden, inter = 512, 1024
    n1 = 2 * inter if gated else inter
    ffn = lt.LeanFFN(
        hidden, inter, gated=gated, layer_norm_eps=1e-5,
        i2h_proj=lt.GeneralizedLinear(lt.GeneralizedMatrix(hidden, n1, None, lowrank_dim), adapter_dim),
        h2o_proj=lt.GeneralizedLinear(lt.GeneralizedMatrix(inter, hidden, None, lowrank_dim), adapter_dim))
    _randomise_small_vectors(ffn)
    with torch.no_grad():
        for proj in (ffn.i2h_proj, ffn.h2o_proj):
            if proj.adapter_second is not None:
                proj.adapter_second.normal_(std=0.05)
            if proj.matrix.lowrank_first is not None:
                proj.matrix.lowrank_first.normal_(std=0.05)
                proj.matrix.lowrank_second.normal_(std=0.05)
    ffn = ffn.to(DEV).to(BF16)
    x, dy = torch.randn(tokens, hidden), torch.randn(tokens, hidden)
    xd = x.to(DEV).requires_grad_(True)
    y = ffn(xd)
    names, params = zip(*ffn.named_parameters())
    grads = torch.autograd.grad(y, [xd, *params], dy.to(DEV))
    ref = _oracle_named_grads(ffn, x, dy)
    y_ref, dx_ref, _ = run_oracle(oracle_params(ffn), x, dy)
    assert_close(y, y_ref, BF16, "y")
    assert_close(grads[0], dx_ref, BF16, "dx")
    for name, grad in zip(names, grads[1:]):
        assert_close(grad, ref[name], BF16, name)


@pytest.mark.parametrize("tokens", [1, 64, 300, 1024])
@pytest.mark.parametrize("lowrank_dim,adapter_dim", [(64, 0), (128, 0), (64, 64)])
@pytest.mark.parametrize("bias", [True, False])
def test_bf16_dense_generalized_linear_alone(tokens, lowrank_dim, adapter_dim, bias):
    """the same layer type on its own (lt_linear_forward / lt_linear_backward), bf16, against fp32 stock ops"""
    torch.manual_seed(tokens + lowrank_dim + adapter_dim)
    fan_in, fan_out = 512, 768
    layer = lt.GeneralizedLinear(lt.GeneralizedMatrix(fan_in, fan_out, None, lowrank_dim), adapter_dim, bias=bias)
    with torch.no_grad():
        if bias:
            layer.bias.normal_(std=0.1)
        if layer.adapter_second is not None:
            layer.adapter_second.normal_(std=0.05)
        layer.matrix.lowrank_first.normal_(std=0.05)
        layer.matrix.lowrank_second.normal_(std=0.05)
    layer = layer.to(DEV).to(BF16)
    x, dy = torch.randn(tokens, fan_in), torch.randn(tokens, fan_out)
    xd = x.to(DEV).to(BF16).requires_grad_(True)
    y = layer(xd)
    names, params = zip(*layer.named_parameters())
    grads = torch.autograd.grad(y, [xd, *params], dy.to(DEV).to(BF16))
    leaves = {n: p.detach().float().cpu().requires_grad_(True) for n, p in layer.named_parameters()}
    xr = x.to(BF16).float().requires_grad_(True)
    firsts = [leaves[k] for k in ("matrix.lowrank_first", "adapter_first") if k in leaves]
    seconds = [leaves[k] for k in ("matrix.lowrank_second", "adapter_second") if k in leaves]
    y_ref = xr @ leaves["matrix.weight"].t() + (xr @ torch.cat(firsts, 0).t()) @ torch.cat(seconds, 1).t()
    if bias:
        y_ref = y_ref + leaves["bias"]
    ref = torch.autograd.grad(y_ref, [xr, *[leaves[n] for n in names]], dy.to(BF16).float())
    assert_close(y, y_ref.detach(), BF16, "y")
    assert_close(grads[0], ref[0], BF16, "dx")
    for name, a, b in zip(names, grads[1:], ref[1:]):
        assert_close(a, b, BF16, name)


def test_in_place_parameter_update_between_forward_and_backward_is_refused():
    """backward reuses fp32 copies of the LayerNorm parameters and biases made in forward; the parameters themselves are
    saved for backward, so updating one in place before backward raises instead of pairing stale copies with fresh weights"""
    ffn = lt.LeanFFN(256, 512, gated=True).to(DEV).to(BF16)
    x = torch.randn(64, 256, device=DEV, dtype=BF16, requires_grad=True)
    y = ffn(x)
    with torch.no_grad():
        ffn.pre_layer_norm.weight.mul_(2.0)
    with pytest.raises(RuntimeError, match="modified by an inplace operation"):
        y.sum().backward()


def _dense_from_native(weight, backward_indices, out_features):
    """[out, in] dense matrix of a native block-sparse weight [in, A, block] (differentiable scatter of its blocks)"""
    in_features, per_in, block = weight.shape
    n_in, n_out = in_features // block, out_features // block
    blocks = weight.reshape(n_in, per_in, block, block)
    grid = torch.zeros(n_out, n_in, block, block, dtype=weight.dtype, device=weight.device)
    ib = torch.arange(n_in, device=weight.device)[:, None].expand(n_in, per_in)
    grid = grid.index_put((backward_indices.to(weight.device), ib), blocks)
    return grid.permute(0, 2, 1, 3).reshape(out_features, in_features)


@pytest.mark.parametrize("tokens", [256, 300, 1024])
@pytest.mark.parametrize("fan_in,fan_out,stretch,run", [(1024, 4096, True, 4), (512, 4096, True, 8), (1024, 4096, False, 1)])
@pytest.mark.parametrize("lowrank_dim", [0, 64])
def test_bf16_blocksparse_layers_with_and_without_shared_list_runs(tokens, fan_in, fan_out, stretch, run, lowrank_dim):
    """a PixelFly layer alone in bf16: stretched over a tall matrix its output blocks come in runs with one list of input
    blocks and the forward product and the weight gradient run as dense products over gathered blocks (whole and partial token
    tiles; token counts that are not a multiple of 32 send the weight gradient back to the walk); tiled, every output block
    has its own list and everything is a walk.  Against fp32 stock ops on the dense expansion of the same weights."""
    from lean_transformer_amd.blocksparse.linear import shared_list_run
    torch.manual_seed(tokens + fan_in + lowrank_dim)
    layout = f"pixelfly(block_size=64, stretch={stretch})"
    layer = lt.GeneralizedLinear(lt.GeneralizedMatrix(fan_in, fan_out, layout, lowrank_dim), bias=True)
    with torch.no_grad():
        layer.bias.normal_(std=0.1)
        layer.weight.normal_(std=0.05)
        if lowrank_dim:
            layer.matrix.lowrank_first.normal_(std=0.05)
            layer.matrix.lowrank_second.normal_(std=0.05)
    layer = layer.to(DEV).to(BF16)
    matrix = layer.matrix
    assert shared_list_run(matrix.forward_indices, matrix.backward_indices.shape[1]) == run
    x, dy = torch.randn(tokens, fan_in), torch.randn(tokens, fan_out)
    xd = x.to(DEV).to(BF16).requires_grad_(True)
    y = layer(xd)
    names, params = zip(*layer.named_parameters())
    grads = torch.autograd.grad(y, [xd, *params], dy.to(DEV).to(BF16))
    leaves = {n: p.detach().float().requires_grad_(True) for n, p in layer.named_parameters()}
    xr = x.to(DEV).to(BF16).float().requires_grad_(True)
    y_ref = xr @ _dense_from_native(leaves["matrix.weight"], matrix.backward_indices, fan_out).t() + leaves["bias"]
    if lowrank_dim:
        y_ref = y_ref + (xr @ leaves["matrix.lowrank_first"].t()) @ leaves["matrix.lowrank_second"].t()
    ref = torch.autograd.grad(y_ref, [xr, *[leaves[n] for n in names]], dy.to(DEV).to(BF16).float())
    assert_close(y, y_ref.detach(), BF16, "y")
    assert_close(grads[0], ref[0], BF16, "dx")
    for name, a, b in zip(names, grads[1:], ref[1:]):
        assert_close(a, b, BF16, name)


@pytest.mark.parametrize("tokens", [256, 300, 1024, 2048])
@pytest.mark.parametrize("fan_in,fan_out,stretch,run", [(4096, 1024, True, 4), (4096, 512, True, 8), (4096, 1024, False, 1)])
@pytest.mark.parametrize("lowrank_dim", [0, 64])
def test_bf16_blocksparse_wide_layers_with_runs_on_the_input_side(tokens, fan_in, fan_out, stretch, run, lowrank_dim):
    """PixelFly stretched over a wide matrix: the input blocks come in runs with one list of output blocks and the weight
    gradient runs as dense products over gathered blocks of dY (2048 tokens: with its reduction over the tokens split in two;
    300 tokens, not a multiple of 32: the walk); tiled, everything is a walk.  Against fp32 stock ops on the dense expansion
    of the same weights."""
    from lean_transformer_amd.blocksparse.linear import shared_input_run, shared_list_run
    torch.manual_seed(tokens + fan_out + lowrank_dim)
    layout = f"pixelfly(block_size=64, stretch={stretch})"
    layer = lt.GeneralizedLinear(lt.GeneralizedMatrix(fan_in, fan_out, layout, lowrank_dim), bias=True)
    with torch.no_grad():
        layer.bias.normal_(std=0.1)
        layer.weight.normal_(std=0.05)
        if lowrank_dim:
            layer.matrix.lowrank_first.normal_(std=0.05)
            layer.matrix.lowrank_second.normal_(std=0.05)
    layer = layer.to(DEV).to(BF16)
    matrix = layer.matrix
    assert shared_input_run(matrix.backward_indices) == run
    assert shared_list_run(matrix.forward_indices, matrix.backward_indices.shape[1]) == 1
    x, dy = torch.randn(tokens, fan_in), torch.randn(tokens, fan_out)
    xd = x.to(DEV).to(BF16).requires_grad_(True)
    y = layer(xd)
    names, params = zip(*layer.named_parameters())
    grads = torch.autograd.grad(y, [xd, *params], dy.to(DEV).to(BF16))
    leaves = {n: p.detach().float().requires_grad_(True) for n, p in layer.named_parameters()}
    xr = x.to(DEV).to(BF16).float().requires_grad_(True)
    y_ref = xr @ _dense_from_native(leaves["matrix.weight"], matrix.backward_indices, fan_out).t() + leaves["bias"]
    if lowrank_dim:
        y_ref = y_ref + (xr @ leaves["matrix.lowrank_first"].t()) @ leaves["matrix.lowrank_second"].t()
    ref = torch.autograd.grad(y_ref, [xr, *[leaves[n] for n in names]], dy.to(DEV).to(BF16).float())
    assert_close(y, y_ref.detach(), BF16, "y")
    assert_close(grads[0], ref[0], BF16, "dx")
    for name, a, b in zip(names, grads[1:], ref[1:]):
        assert_close(a, b, BF16, name)


@pytest.mark.parametrize("gated", [False, True])
@pytest.mark.parametrize("tokens", [512, 300])
def test_bf16_ffn_with_blocksparse_projections_in_runs(gated, tokens):
    """LeanFFN whose up-projection is PixelFly stretched over a tall matrix (runs of output blocks with one list): plain GELU
    takes the dense product's fused activation epilogue, GeGLU the product and the activation pass"""
    torch.manual_seed(tokens + gated)
    hidden, inter = 512, 2048
    layout = "pixelfly(block_size=64, stretch=True)"
    up = lt.GeneralizedLinear(lt.GeneralizedMatrix(hidden, inter * (2 if gated else 1), layout, 64))
    down = lt.GeneralizedLinear(lt.GeneralizedMatrix(inter, hidden, layout, 64))
    ffn = lt.LeanFFN(hidden, inter, gated=gated, i2h_proj=up, h2o_proj=down)
    _randomise_small_vectors(ffn)
    with torch.no_grad():
        for t in (up.weight, down.weight, up.matrix.lowrank_first, up.matrix.lowrank_second, down.matrix.lowrank_first,
                  down.matrix.lowrank_second):
            t.normal_(std=0.05)
    ffn = ffn.to(DEV).to(BF16)
    x, dy = torch.randn(tokens, hidden), torch.randn(tokens, hidden)
    _compare(ffn, x.to(BF16), dy.to(BF16), BF16)


@pytest.mark.parametrize("sparse", [False, True])
def test_repeated_steps_are_bitwise_identical(sparse):
    """no kernel on the path sums in an order that depends on scheduling (split reductions are summed in slice order, column
    sums per fixed row slices, no atomics): the same step twice gives the same bits in y and in every gradient"""
    torch.manual_seed(5)
    hidden, inter = 512, 2048
    if sparse:
        layout = "pixelfly(block_size=64, stretch=True)"
        up = lt.GeneralizedLinear(lt.GeneralizedMatrix(hidden, 2 * inter, layout, 64))
        down = lt.GeneralizedLinear(lt.GeneralizedMatrix(inter, hidden, layout, 64))
        ffn = lt.LeanFFN(hidden, inter, gated=True, i2h_proj=up, h2o_proj=down, dropout=0.1)
    else:
        ffn = lt.LeanFFN(hidden, inter, gated=True, dropout=0.1)
    ffn = ffn.to(DEV).to(BF16).train()
    x = torch.randn(1024, hidden, device=DEV, dtype=BF16, requires_grad=True)
    dy = torch.randn(1024, hidden, device=DEV, dtype=BF16)
    params = list(ffn.parameters())
    runs = []
    for _ in range(2):
        torch.manual_seed(11)  # same dropout stream
        y = ffn(x)
        runs.append([y.detach().clone()] + [g.clone() for g in torch.autograd.grad(y, [x, *params], dy)])
    for a, b in zip(*runs):
        assert torch.equal(a, b)
