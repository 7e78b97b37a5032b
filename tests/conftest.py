import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def golden_dir():
    return os.path.join(ROOT, "tests", "golden")


class Checkpoint:
    """A seeded synthetic checkpoint written twice as a weight directory: `raw` as drawn
    (float32) and `bf16x` with the Linear kernels rounded to bfloat16-representable values.
    `npy_raw` / `npy_bf16x` are the same tensors in the on-disk layout, for the oracle."""

    def __init__(self, root, dims, seed, degenerate):
        from cudabert_amd import weights as W
        self.dims = dims
        state = W.synth_state(dims, seed=seed, degenerate=degenerate)
        self.raw = W.export_npy_dir(state, str(root / "raw"))
        self.npy_raw = W.to_npy_layout(state)
        state = W.bf16_representable(state)
        self.bf16x = W.export_npy_dir(state, str(root / "bf16x"))
        self.npy_bf16x = W.to_npy_layout(state)

    def dir(self, exact):
        return self.bf16x if exact else self.raw

    def npy(self, exact):
        return self.npy_bf16x if exact else self.npy_raw


@pytest.fixture(scope="session")
def large_ckpt(tmp_path_factory):
    """BERT-large with the stock initialisation and the benchmark's seed: the checkpoint
    bench.py runs."""
    from cudabert_amd import weights as W
    return Checkpoint(tmp_path_factory.mktemp("large"), W.LARGE, 20240, True)


@pytest.fixture(scope="session")
def base_ckpt(tmp_path_factory):
    from cudabert_amd import weights as W
    return Checkpoint(tmp_path_factory.mktemp("base"), W.BASE, 20240, True)
