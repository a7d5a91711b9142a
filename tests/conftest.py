import sys
from pathlib import Path

import numpy as np
import pytest
import torch

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

GOLDEN = ROOT / "tests" / "golden" / "attention_golden.npz"

# Parity bar for a bf16 kernel against the fp32 reference.
MAX_ABS_TOL = 2e-2
MEAN_ABS_TOL = 2e-3


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


class GoldenCase:
    """One known-answer vector: tensors (bf16 inputs restored from their bit patterns), expected fp32 output, meta."""

    def __init__(self, name, arrays):
        self.name = name
        self.inputs, self.meta = {}, {}
        for key, arr in arrays.items():
            if key == "expected":
                self.expected = torch.from_numpy(arr)
            elif key.startswith("meta."):
                self.meta[key[5:]] = arr.item()
            elif key.endswith(".bf16"):
                self.inputs[key[:-5]] = torch.from_numpy(arr.view(np.int16).copy()).view(torch.bfloat16)
            else:
                self.inputs[key] = torch.from_numpy(arr)

    def to(self, device, dtype=None):
        out = {}
        for k, t in self.inputs.items():
            t = t.to(device)
            if dtype is not None and t.is_floating_point():
                t = t.to(dtype)
            out[k] = t
        return out


def load_golden():
    data = np.load(GOLDEN)
    cases = {}
    for key in data.files:
        name, field = key.split("/", 1)
        cases.setdefault(name, {})[field] = data[key]
    return {n: GoldenCase(n, a) for n, a in cases.items()}


@pytest.fixture(scope="session")
def golden():
    return load_golden()


def assert_parity(out: torch.Tensor, ref: torch.Tensor, what: str = "", max_tol=MAX_ABS_TOL, mean_tol=MEAN_ABS_TOL):
    assert tuple(out.shape) == tuple(ref.shape), f"{what}: shape {tuple(out.shape)} vs {tuple(ref.shape)}"
    o = out.detach().float().cpu()
    r = ref.detach().float().cpu()
    assert torch.isfinite(o).all(), f"{what}: non-finite output"
    d = (o - r).abs()
    mx, mn = d.max().item(), d.mean().item()
    assert mx <= max_tol and mn <= mean_tol, f"{what}: max-abs {mx:.3e} (tol {max_tol}), mean-abs {mn:.3e} (tol {mean_tol})"
    return mx, mn
