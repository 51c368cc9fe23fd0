import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an AMD GPU (run on the MI355X box); everything else runs on CPU")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


def rel_err(got: torch.Tensor, ref: torch.Tensor) -> float:
    """max |got - ref| / max |ref|: the "max relative error" of the parity bar (fp32 <= 1e-4, bf16 <= 2e-2)"""
    got, ref = got.detach().double().cpu(), ref.detach().double().cpu()
    denom = ref.abs().max().item()
    return (got - ref).abs().max().item() / (denom if denom > 0 else 1.0)


def cosine(got: torch.Tensor, ref: torch.Tensor) -> float:
    got, ref = got.detach().double().cpu().flatten(), ref.detach().double().cpu().flatten()
    denom = (got.norm() * ref.norm()).item()
    return (got @ ref).item() / denom if denom > 0 else 1.0


FP32_TOL = 1e-4   # max relative error, fp32 path
BF16_TOL = 2e-2   # max relative error, bf16 path
BF16_COS = 0.9999  # minimum cosine similarity, bf16 path


def assert_close(got, ref, dtype, name=""):
    assert got.shape == ref.shape, f"{name}: shape {tuple(got.shape)} vs {tuple(ref.shape)}"
    assert torch.isfinite(got.float()).all(), f"{name}: non-finite values"
    err = rel_err(got, ref)
    if dtype == torch.float32:
        assert err <= FP32_TOL, f"{name}: max relative error {err:.3e} > {FP32_TOL}"
        # element by element as well, in the form of the reference's own fp32 checks (tests/test_ffn.py:175, allclose with
        # rtol 1e-4, atol 1e-5), the absolute floor scaled to the tensor's magnitude so that small entries are not hidden
        g, r = got.detach().double().cpu(), ref.detach().double().cpu()
        floor = 1e-5 * max(r.abs().max().item(), 1e-30)
        worst = ((g - r).abs() - (1e-4 * r.abs() + floor)).max().item() if r.numel() else 0.0
        assert worst <= 0.0, f"{name}: an element is {worst:.3e} beyond 1e-4 * |ref| + 1e-5 * max|ref|"
    else:
        cos = cosine(got, ref)
        assert err <= BF16_TOL and cos >= BF16_COS, f"{name}: max relative error {err:.3e}, cosine {cos:.6f}"
