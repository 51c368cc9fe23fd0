"""Checkpoint interop on the GPU: a state_dict written by modules that share no class with lean_transformer_amd (the
reference tests' look-alike pattern, tests/test_ffn.py:89-147,199), saved to disk under the reference's older key names
without the `.layout` buffers, read back with a weights-only loader, loaded into LeanFFN with PixelFly projections + shared
low-rank term + adapter, and run on the HIP kernels against the look-alike's stock-op forward and autograd."""
import pytest
import torch

import lean_transformer_amd as lt
from conftest import assert_close
from lookalike import LookAlikeFFN, LookAlikeLinear, LookAlikeMatrix

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

_TO_LEGACY = ((".matrix.", ".shared_matrix."), (".i2h_proj", ".dense_i2h"), (".h2o_proj", ".dense_h2o"),
              ("ffn.pre_layer_norm", "ffn.layer_norm"), (".post_layer_norm", ".sandwich_norm"))


@pytest.mark.parametrize("dtype,hidden,inter,block", [(torch.float32, 64, 128, 16), (torch.bfloat16, 256, 512, 64)])
@pytest.mark.parametrize("legacy_names", [False, True])
def test_lookalike_checkpoint_loads_and_matches(tmp_path, dtype, hidden, inter, block, legacy_names):
    torch.manual_seed(hidden + legacy_names)
    src = LookAlikeFFN(hidden, inter, True, LookAlikeLinear(LookAlikeMatrix(hidden, 2 * inter, block, 8), 4),
                       LookAlikeLinear(LookAlikeMatrix(inter, hidden, block, 8), 4), post_layer_norm=True)
    with torch.no_grad():
        for ln in (src.pre_layer_norm, src.post_layer_norm):
            ln.weight.uniform_(0.5, 1.5)
            ln.bias.normal_(std=0.2)
    state = {"ffn." + k: v for k, v in src.state_dict().items()}
    if legacy_names:
        renamed = {}
        for key, value in state.items():
            if key.endswith(".layout"):
                continue  # older checkpoints did not store it
            for new, old in _TO_LEGACY:
                key = key.replace(new, old)
            renamed[key] = value
        state = renamed
    path = tmp_path / "ffn.pth"
    torch.save(state, path)
    loaded = torch.load(path, weights_only=True)

    class Host(torch.nn.Module):
        def __init__(self):
            super().__init__()
            layout = f"pixelfly(block_size={block})"
            up = lt.GeneralizedLinear(lt.GeneralizedMatrix(hidden, 2 * inter, layout, lowrank_dim=8), adapter_dim=4)
            down = lt.GeneralizedLinear(lt.GeneralizedMatrix(inter, hidden, layout, lowrank_dim=8), adapter_dim=4)
            self.ffn = lt.LeanFFN(hidden, inter, gated=True, post_layer_norm=True, layer_norm_eps=1e-5, i2h_proj=up,
                                  h2o_proj=down)

    host = Host()
    report = lt.load_reference_state_dict(host, loaded)
    assert not report.missing_keys and not report.unexpected_keys
    ffn = host.ffn.to(DEV).to(dtype)
    if dtype == torch.bfloat16:  # the look-alike computes in fp32 on the weights as the kernels see them
        with torch.no_grad():
            for p in src.parameters():
                p.copy_(p.to(torch.bfloat16).float())
    x, dy = torch.randn(3, 50, hidden), torch.randn(3, 50, hidden)
    xr = x.clone().requires_grad_(True)
    names, ref_params = zip(*src.named_parameters())
    y_ref = src(xr)
    ref = torch.autograd.grad(y_ref, [xr, *ref_params], dy)
    xd = x.to(DEV).requires_grad_(True)
    y = ffn(xd)
    own = dict(ffn.named_parameters())
    got = torch.autograd.grad(y, [xd, *[own[n] for n in names]], dy.to(DEV))
    assert_close(y, y_ref.detach(), dtype, "y")
    assert_close(got[0], ref[0], dtype, "dx")
    for name, a, b in zip(names, got[1:], ref[1:]):
        assert_close(a, b, dtype, name)
