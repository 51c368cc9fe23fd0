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
FP16_TOL = 4e-3   # max relative error, fp16 path (11 significant bits against bf16's 8: the bf16 bar / 5)
FP16_COS = 0.999996  # minimum cosine similarity, fp16 path (1 - cosine goes with the square of the error: 1e-4 / 25)


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
        tol, floor = (FP16_TOL, FP16_COS) if dtype == torch.float16 else (BF16_TOL, BF16_COS)
        assert err <= tol and cos >= floor, f"{name}: max relative error {err:.3e} (bar {tol}), cosine {cos:.7f} (bar {floor})"


def assert_within_bf16_noise(named_got, named_truth, stock_runs, label="", depth=1):
    """Deep bf16 computations (a module applied several times in a row, a whole model): rounding noise compounds, so two
    equally valid bf16 runs differ from the fp32 truth -- and from each other -- by more than the single-application bar.
    `named_got` / `named_truth`: {name: tensor}; `stock_runs`: two or more {name: tensor} results of stock-op bf16 runs of the
    same computation; `depth`: how many applications of the block follow one another.  A tensor passes when it meets the bar
    of one application (max relative error 2e-2, cosine 0.9999) scaled to `depth` independent applications -- errors add in
    quadrature, so 2e-2 sqrt(depth), and 1 - cosine, which goes with the square of the error, 1e-4 depth -- or when both
    figures are within 1.1 x swing x the largest of the stock-op runs' figures, swing being the largest factor by which that
    figure moves on any tensor between two stock-op runs (measured here, per figure)."""
    assert len(stock_runs) >= 2
    figures = {name: [(rel_err(run[name], truth), 1.0 - cosine(run[name], truth)) for run in stock_runs]
               for name, truth in named_truth.items()}
    swing_err = max(max(e for e, _ in f) / max(min(e for e, _ in f), 1e-12) for f in figures.values())
    swing_ang = max(max(a for _, a in f) / max(min(a for _, a in f), 1e-12) for f in figures.values())
    failures = []
    for name, truth in named_truth.items():
        got = named_got[name]
        assert got.shape == truth.shape and torch.isfinite(got.float()).all(), name
        err, ang = rel_err(got, truth), 1.0 - cosine(got, truth)
        if err <= BF16_TOL * depth ** 0.5 and ang <= (1.0 - BF16_COS) * depth:
            continue
        e_max, a_max = max(e for e, _ in figures[name]), max(a for _, a in figures[name])
        if err > 1.1 * swing_err * e_max or ang > 1.1 * swing_ang * a_max:
            failures.append(f"{name}: max relative error {err:.3e} (stock-op bf16 runs " + " ".join(f"{e:.3e}" for e, _ in figures[name])
                            + f", swing {swing_err:.2f}), 1 - cosine {ang:.3e} (" + " ".join(f"{a:.3e}" for _, a in figures[name])
                            + f", swing {swing_ang:.2f})")
    assert not failures, label + "\n" + "\n".join(failures)
