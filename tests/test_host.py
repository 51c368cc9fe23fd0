"""Host-side logic of the product package, on CPU: layouts / index tables against the reference's golden vectors, the module
API and state_dict contract, activation mapping, and that the C-ABI library loads and exports what include/leanffn.h declares.
No kernel is launched here."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch
import torch.nn as nn

import lean_transformer_amd as lt
from lean_transformer_amd import _native as nat
from lean_transformer_amd.blocksparse import layout as lay
from lean_transformer_amd.utils import ACT2FN, activation_kind
from oracle import ffn as offn

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLDEN = np.load(os.path.join(os.path.dirname(__file__), "golden", "blocksparse_golden.npz"))


@pytest.mark.parametrize("name", [str(n) for n in GOLDEN["names"]])
def test_layout_and_indices_match_reference_golden(name):
    out_f, in_f, block = (int(v) for v in GOLDEN[f"{name}/shape"])
    layout = lay.get_blocksparse_layout(out_f, in_f, str(GOLDEN[f"{name}/desc"]))
    assert layout.dtype == torch.bool and np.array_equal(layout.numpy(), GOLDEN[f"{name}/layout"])
    fwd, bwd = lay.get_indices_from_layout(layout)
    assert fwd.dtype == torch.int32 and bwd.dtype == torch.int64
    assert np.array_equal(fwd.numpy(), GOLDEN[f"{name}/forward_indices"])
    assert np.array_equal(bwd.numpy(), GOLDEN[f"{name}/backward_indices"])


def test_layout_headline_shape_without_element_mask():
    """32768 x 4096 with 64 x 64 blocks: 7 active blocks per row of the 64-cell butterfly, stretched or tiled"""
    for stretch in (True, False):
        up = lay.get_blocksparse_layout(32768, 4096, f"pixelfly(block_size=64, stretch={stretch})")
        down = lay.get_blocksparse_layout(4096, 16384, f"pixelfly(block_size=64, stretch={stretch})")
        assert up.shape == (512, 64) and down.shape == (64, 256)
        assert up.sum(1).unique().tolist() == [7] and up.sum(0).unique().tolist() == [56]
        assert down.sum(1).unique().tolist() == [28] and down.sum(0).unique().tolist() == [7]
        fwd, bwd = lay.get_indices_from_layout(up)
        assert fwd.shape == (512, 7) and bwd.shape == (64, 56) and fwd.max() == 7 * 512 - 1


def test_layout_registry_and_errors():
    @lay.register_blocksparse_layout("test_diag")
    def make(out_features, in_features, foo):
        smaller = min(out_features, in_features)
        eye = torch.eye(smaller // foo, dtype=torch.bool)
        return eye.repeat(out_features // smaller, in_features // smaller)

    assert lay.get_blocksparse_layout(64, 32, "test_diag(foo=4)").float().mean().item() == pytest.approx(0.125)
    with pytest.raises(ValueError):
        lay.get_blocksparse_layout(64, 64, "nonexistent(1)")
    with pytest.raises(AssertionError):
        lay.get_indices_from_layout(torch.tensor([[True, False], [True, True]]))  # unbalanced
    lay.REGISTERED_LAYOUTS.pop("test_diag")


def test_constructor_defaults_and_state_dict_keys():
    ffn = lt.LeanFFN(32, 128)
    assert isinstance(ffn.i2h_proj, nn.Linear) and ffn.i2h_proj.out_features == 128
    assert (ffn.gated, ffn.dropout, ffn.residual, ffn.ffn_custom_grad, ffn.post_layer_norm) == (False, 0.0, True, True, None)
    assert ffn.pre_layer_norm.eps == 1e-12 and ffn.activation is ACT2FN["gelu_fused"]
    assert sorted(ffn.state_dict()) == ["h2o_proj.bias", "h2o_proj.weight", "i2h_proj.bias", "i2h_proj.weight",
                                        "pre_layer_norm.bias", "pre_layer_norm.weight"]
    gated = lt.LeanFFN(32, 128, gated=True, post_layer_norm=True)
    assert gated.i2h_proj.out_features == 256 and "post_layer_norm.weight" in gated.state_dict()
    with pytest.raises(AssertionError):
        lt.LeanFFN(32, 128, i2h_proj=nn.Linear(32, 64))
    with pytest.raises(AssertionError):
        lt.LeanFFN(32, 128, i2h_proj=nn.Sequential(nn.Linear(32, 128)))


def test_generalized_linear_parameter_layout():
    matrix = lt.GeneralizedMatrix(32, 256, "pixelfly(16)", lowrank_dim=4)
    lin = lt.GeneralizedLinear(matrix, adapter_dim=2)
    assert lin.weight is matrix.weight and tuple(matrix.weight.shape) == (32, 16, 16)
    assert tuple(matrix.lowrank_first.shape) == (4, 32) and tuple(matrix.lowrank_second.shape) == (256, 4)
    first, second = lin.get_combined_lowrank_components()
    assert tuple(first.shape) == (6, 32) and tuple(second.shape) == (256, 6)
    assert sorted(lin.state_dict()) == ["adapter_first", "adapter_second", "bias", "matrix.backward_indices",
                                        "matrix.forward_indices", "matrix.layout", "matrix.lowrank_first",
                                        "matrix.lowrank_second", "matrix.weight"]
    dense = lt.GeneralizedLinear(lt.GeneralizedMatrix(32, 64))
    assert tuple(dense.weight.shape) == (64, 32) and dense.matrix.forward_indices is None
    assert dense.get_combined_lowrank_components() == (None, None)
    with pytest.raises(NotImplementedError):
        lt.GeneralizedMatrix(32, 64, "pixelfly(16)", blocksparse_backend="triton")
    # a matrix shared between two layers is one parameter
    shared = lt.GeneralizedMatrix(32, 32)
    a, b = lt.GeneralizedLinear(shared, 2), lt.GeneralizedLinear(shared, 2)
    assert a.weight is b.weight and a.adapter_first is not b.adapter_first


def test_checkpoint_round_trip_in_the_reference_key_layout(tmp_path):
    """A checkpoint written from the module holds exactly the keys the reference's module would write (nn.Linear:
    ffn.py:51-52; GeneralizedLinear: blocksparse/linear.py:32-66, 109-123, layout and index tables as persistent buffers)
    and loads back strictly, from a file read with weights_only=True, into a freshly constructed module."""
    torch.manual_seed(0)

    def sparse_ffn():
        up = lt.GeneralizedLinear(lt.GeneralizedMatrix(32, 256, "pixelfly(16)", lowrank_dim=4), adapter_dim=2)
        down = lt.GeneralizedLinear(lt.GeneralizedMatrix(128, 32, "pixelfly(16)", lowrank_dim=4), adapter_dim=2)
        return lt.LeanFFN(32, 128, gated=True, i2h_proj=up, h2o_proj=down)

    for make in (lambda: lt.LeanFFN(32, 128, gated=True, post_layer_norm=True), sparse_ffn):
        src, dst = make(), make()
        with torch.no_grad():
            for t in src.parameters():
                t.normal_()
        path = tmp_path / "ffn.pth"
        torch.save(src.state_dict(), path)
        state = torch.load(path, weights_only=True)
        assert list(state) == list(src.state_dict())
        result = dst.load_state_dict(state, strict=True)
        assert not result.missing_keys and not result.unexpected_keys
        for key, value in src.state_dict().items():
            assert torch.equal(dst.state_dict()[key], value) and dst.state_dict()[key].dtype == value.dtype, key
    sparse = sparse_ffn().state_dict()
    assert sparse["i2h_proj.matrix.layout"].dtype == torch.bool and tuple(sparse["i2h_proj.matrix.layout"].shape) == (16, 2)
    assert sparse["i2h_proj.matrix.forward_indices"].dtype == torch.int32
    assert sparse["i2h_proj.matrix.backward_indices"].dtype == torch.int64
    assert tuple(sparse["i2h_proj.matrix.weight"].shape) == (32, 16, 16)  # native order [in_features, A, block]


def test_activation_mapping():
    assert activation_kind(ACT2FN["gelu_fused"]) == "gelu_fused"
    assert activation_kind(ACT2FN["gelu_new"]) == "gelu_fused"
    assert activation_kind(ACT2FN["relu"]) == "relu" and activation_kind(ACT2FN["swish"]) == "silu"
    assert activation_kind(torch.nn.functional.gelu) == "gelu" and activation_kind(nn.GELU(approximate="tanh")) == "gelu_fused"
    assert activation_kind(torch.sigmoid) == "sigmoid" and activation_kind(nn.LeakyReLU()) == "leaky_relu"
    with pytest.raises(NotImplementedError):
        activation_kind(torch.exp)
    x = torch.linspace(-5, 5, 1000)
    assert (ACT2FN["gelu_fused"](x) - torch.nn.functional.gelu(x)).abs().max().item() <= 5e-4  # reference tests/test_utils.py:25-29
    assert torch.allclose(ACT2FN["gelu_fused"](x), offn.gelu_fused(x))


def test_plain_autograd_path_on_cpu_matches_oracle():
    """ffn_custom_grad=False is the reference's stock-op composition (ffn.py:69-85); with nn.Linear projections it runs
    anywhere and must equal the oracle's plain_ffn"""
    torch.manual_seed(0)
    ffn = lt.LeanFFN(16, 32, gated=True, post_layer_norm=True, layer_norm_eps=1e-5, ffn_custom_grad=False)
    x = torch.randn(2, 3, 16)
    p = offn.FFNParams(ffn.pre_layer_norm.weight, ffn.pre_layer_norm.bias,
                       offn.LinearParams(ffn.i2h_proj.weight, ffn.i2h_proj.bias, out_features=64),
                       offn.LinearParams(ffn.h2o_proj.weight, ffn.h2o_proj.bias, out_features=16),
                       ffn.post_layer_norm.weight, ffn.post_layer_norm.bias,
                       offn.FFNConfig(gated=True, ln_eps=1e-5))
    assert torch.allclose(ffn(x), offn.plain_ffn(x, p), rtol=1e-5, atol=1e-6)


def test_custom_path_refuses_cpu_tensors():
    ffn = lt.LeanFFN(16, 32)
    with pytest.raises(RuntimeError, match="AMD GPUs only"):
        ffn(torch.randn(2, 16))
    with pytest.raises(RuntimeError, match="AMD GPUs only"):
        lt.blocksparse_matmul(torch.randn(2, 8), torch.randn(8, 2, 2), torch.zeros(4, 2, dtype=torch.int32))


def test_library_loads_and_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "leanffn.h")).read()
    declared = set(re.findall(r"\b(lt_[a-z0-9_]+)\s*\(", header))
    assert declared == set(nat.EXPORTED_SYMBOLS), declared ^ set(nat.EXPORTED_SYMBOLS)
    for dtype, half in ((torch.bfloat16, "bf16"), (torch.float16, "fp16")):  # the library and its float16 twin
        lib = nat.lib(dtype)
        for name in declared:
            assert hasattr(lib, name), name
        version = lib.lt_version().decode()
        assert version.startswith("libleanffn") and half in version, version
    assert nat.lib() is nat.lib(torch.float32) is nat.lib(torch.bfloat16) is not nat.lib(torch.float16)
    with pytest.raises(TypeError, match="one 16-bit type"):
        nat.lib(torch.float16, torch.bfloat16)


def test_struct_layouts_match_header_sizes():
    # pointer-sized and 4-byte members only: sizes are fixed by the C ABI on x86-64
    assert ctypes.sizeof(nat.LtLinear) == 6 * 8 + 8 * 4
    assert ctypes.sizeof(nat.LtLinearGrads) == 32
    assert ctypes.sizeof(nat.LtFfnSaved) == 40
    assert ctypes.sizeof(nat.LtFfnGrads) == 5 * 8 + 2 * 32
    assert ctypes.sizeof(nat.LtFfnDesc) == 8 + 7 * 4 + 2 * 4 + 2 * 8 + 4 * 8 + 2 * ctypes.sizeof(nat.LtLinear) + 4


def test_argument_errors_are_reported_not_crashed():
    lib = nat.lib()
    desc = nat.LtFfnDesc()  # all zero
    assert lib.lt_ffn_forward_workspace_bytes(desc) == 0
    status = lib.lt_ffn_forward(desc, None, None, nat.LtFfnSaved(), None, 0, None)
    assert status == 1 and b"bad sizes" in lib.lt_last_error()
    with pytest.raises(RuntimeError, match="lt_status 1"):
        nat.check(status, "lt_ffn_forward")


def test_legacy_checkpoint_keys_and_missing_layout_buffers(tmp_path):
    """A checkpoint in the reference's older naming (the substitutions of reference tests/test_gpt_exact_match.py:51-80),
    without the `.layout` buffers those checkpoints lacked, written by a module that shares no class with this package,
    read back with weights_only=True and loaded through load_reference_state_dict."""
    from lookalike import LookAlikeFFN, LookAlikeLinear, LookAlikeMatrix
    torch.manual_seed(0)
    hidden, inter = 64, 128
    src = LookAlikeFFN(hidden, inter, True, LookAlikeLinear(LookAlikeMatrix(hidden, 2 * inter, 16, 4), 2),
                       LookAlikeLinear(LookAlikeMatrix(inter, hidden, 16, 4), 2), post_layer_norm=True)
    legacy = {}
    for key, value in src.state_dict().items():
        if key.endswith(".layout"):
            continue
        key = "ffn." + key
        for new, old in ((".matrix.", ".shared_matrix."), (".i2h_proj", ".dense_i2h"), (".h2o_proj", ".dense_h2o"),
                         ("ffn.pre_layer_norm", "ffn.layer_norm"), (".post_layer_norm", ".sandwich_norm")):
            key = key.replace(new, old)
        legacy[key[len("ffn."):]] = value
    assert "dense_i2h.shared_matrix.weight" in legacy and "sandwich_norm.weight" in legacy and "layer_norm.bias" in legacy
    path = tmp_path / "legacy.pth"
    torch.save(legacy, path)
    state = torch.load(path, weights_only=True)
    converted = lt.convert_legacy_state_dict({"ffn." + k: v for k, v in state.items()})
    assert "ffn.i2h_proj.matrix.weight" in converted and "ffn.pre_layer_norm.bias" in converted

    def make():
        up = lt.GeneralizedLinear(lt.GeneralizedMatrix(hidden, 2 * inter, "pixelfly(16)", lowrank_dim=4), adapter_dim=2)
        down = lt.GeneralizedLinear(lt.GeneralizedMatrix(inter, hidden, "pixelfly(16)", lowrank_dim=4), adapter_dim=2)
        return lt.LeanFFN(hidden, inter, gated=True, post_layer_norm=True, layer_norm_eps=1e-5, i2h_proj=up, h2o_proj=down)

    class Wrapper(nn.Module):  # the legacy renames are written for keys inside a model ("...ffn.layer_norm")
        def __init__(self):
            super().__init__()
            self.ffn = make()

    dst = Wrapper()
    report = lt.load_reference_state_dict(dst, {"ffn." + k: v for k, v in state.items()})
    assert not report.missing_keys and not report.unexpected_keys
    for key, value in src.state_dict().items():
        assert torch.equal(dst.ffn.state_dict()[key], value), key
    # a checkpoint written for another layout is refused instead of scattering its blocks to the wrong places
    other = LookAlikeFFN(hidden, inter, True, LookAlikeLinear(LookAlikeMatrix(hidden, 2 * inter, 16, 4, stretch=True), 2),
                         LookAlikeLinear(LookAlikeMatrix(inter, hidden, 16, 4), 2), post_layer_norm=True)
    with pytest.raises(ValueError):
        lt.load_reference_state_dict(make(), other.state_dict())
    with pytest.raises(RuntimeError):
        lt.load_reference_state_dict(make(), {k: v for k, v in src.state_dict().items() if "adapter" not in k})


def test_native_and_block_list_weight_orders():
    """native [in, A, block] <-> row-major list of [block, block] sub-matrices, against the oracle's dense expansion"""
    from oracle import blocksparse as obs
    torch.manual_seed(1)
    for out_f, in_f, block, stretch in ((256, 64, 16, False), (64, 256, 16, True), (128, 128, 8, False)):
        m = lt.GeneralizedMatrix(in_f, out_f, f"pixelfly({block}, stretch={stretch})")
        w = m.weight.detach()
        blocks, coords = lt.native_to_block_list(w, m.backward_indices, out_f)
        dense = obs.sparse_to_dense(w, m.backward_indices.numpy(), out_f)
        nz = m.layout.nonzero()
        assert torch.equal(coords, nz)  # row-major order of the layout's active blocks
        for n, (ob, ib) in enumerate(coords.tolist()):
            assert torch.equal(blocks[n], dense[ob * block:(ob + 1) * block, ib * block:(ib + 1) * block])
        assert torch.equal(lt.block_list_to_native(blocks, coords, m.backward_indices), w)
        perm = torch.randperm(len(blocks))
        assert torch.equal(lt.block_list_to_native(blocks[perm], coords[perm], m.backward_indices), w)
    with pytest.raises(ValueError):
        lt.block_list_to_native(blocks, coords.flip(1), m.backward_indices[:, :1])


def test_shared_input_run_of_pixelfly_layouts():
    """runs of consecutive input blocks with one list of output blocks: stretched PixelFly on a wide matrix repeats every list
    in_blocks / out_blocks times; tall, square and tiled layouts have none; the cached value follows in-place changes"""
    from lean_transformer_amd.blocksparse.linear import shared_input_run
    for out_f, in_f, stretch, expected in [(1024, 4096, True, 4), (512, 4096, True, 8), (1024, 4096, False, 1),
                                           (1024, 1024, True, 1), (4096, 1024, True, 1)]:
        layout = lt.get_blocksparse_layout(out_f, in_f, f"pixelfly(block_size=64, stretch={stretch})")
        _, backward_indices = lt.get_indices_from_layout(layout)
        assert shared_input_run(backward_indices) == expected, (out_f, in_f, stretch)
    _, backward_indices = lt.get_indices_from_layout(lt.get_blocksparse_layout(1024, 4096, "pixelfly(block_size=64, stretch=True)"))
    assert shared_input_run(backward_indices) == 4
    backward_indices[1] = backward_indices[8]
    assert shared_input_run(backward_indices) == 1


def test_strided_runs_of_tiled_pixelfly_layouts():
    """PixelFly with stretch=False tiles the square butterfly: blocks one square width apart share their lists.  The group
    value for the C ABI carries the number of such blocks in its low 16 bits and their distance in the high 16 bits; stretched
    layouts keep their plain run length; square ones have neither"""
    from lean_transformer_amd.blocksparse.linear import shared_input_group, shared_list_group
    for out_f, in_f, stretch, out_group, in_group in [
            (4096, 1024, False, 4 | (16 << 16), 1), (1024, 4096, False, 1, 4 | (16 << 16)), (4096, 512, False, 8 | (8 << 16), 1),
            (4096, 1024, True, 4, 1), (1024, 4096, True, 1, 4), (1024, 1024, False, 1, 1)]:
        layout = lt.get_blocksparse_layout(out_f, in_f, f"pixelfly(block_size=64, stretch={stretch})")
        forward_indices, backward_indices = lt.get_indices_from_layout(layout)
        assert shared_list_group(forward_indices, backward_indices.shape[1]) == out_group, (out_f, in_f, stretch)
        assert shared_input_group(backward_indices) == in_group, (out_f, in_f, stretch)


def test_shared_list_run_of_pixelfly_layouts():
    """runs of consecutive output blocks with one list of input blocks: stretched PixelFly on a tall matrix repeats every list
    out_blocks / in_blocks times, the tiled form and square matrices have none; the cached value follows in-place changes"""
    from lean_transformer_amd.blocksparse.linear import shared_list_run
    for out_f, in_f, stretch, expected in [(4096, 1024, True, 4), (4096, 512, True, 8), (4096, 1024, False, 1),
                                           (1024, 1024, True, 1), (1024, 4096, True, 1)]:
        layout = lt.get_blocksparse_layout(out_f, in_f, f"pixelfly(block_size=64, stretch={stretch})")
        forward_indices, backward_indices = lt.get_indices_from_layout(layout)
        assert shared_list_run(forward_indices, backward_indices.shape[1]) == expected, (out_f, in_f, stretch)
    layout = lt.get_blocksparse_layout(4096, 1024, "pixelfly(block_size=64, stretch=True)")
    forward_indices, backward_indices = lt.get_indices_from_layout(layout)
    per_in = backward_indices.shape[1]
    assert shared_list_run(forward_indices, per_in) == 4
    forward_indices[1] = forward_indices[8]  # output block 1 now reads other input blocks than 0, 2 and 3
    assert shared_list_run(forward_indices, per_in) == 1
