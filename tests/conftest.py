import sys
from pathlib import Path

import numpy as np
import pytest

ROOT = Path(__file__).resolve().parents[1]
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a ROCm GPU (MI355X); run with -m gpu")


def bf16_words(values):
    """float -> BF16 bit patterns, round to nearest even."""
    u = np.ascontiguousarray(values, dtype=np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def words_to_float(words):
    return (np.asarray(words).astype(np.uint32) << 16).view(np.float32)


SPECIAL_WORDS = np.array([0, 0x8000, 0x7F80, 0xFF80, 0x7FC1, 0xFFE5, 1, 0x8001], dtype=np.uint16)


def weight_like(rng, rows, cols, sigma=0.02, row_scale=True, outliers=True):
    """Synthetic BF16 weights: N(0, sigma) with per-row log-normal scale and 0.1% outliers at 10x."""
    w = rng.normal(0.0, sigma, size=(rows, cols)).astype(np.float32)
    if row_scale:
        w *= rng.lognormal(0.0, 0.5, size=(rows, 1)).astype(np.float32)
    if outliers:
        w = np.where(rng.random((rows, cols)) < 1e-3, w * 10.0, w).astype(np.float32)
    return bf16_words(w)


@pytest.fixture(scope="session")
def oracle():
    from oracle import codec_oracle
    codec_oracle.lib()
    return codec_oracle
