"""Shared test helpers: seeded synthetic inputs and golden-vector loading."""
import json
from pathlib import Path

import numpy as np

GOLDEN = Path(__file__).resolve().parent / "golden"


def golden_vectors():
    return json.loads((GOLDEN / "reference_vectors.json").read_text())


def synth_weights(rng, n, k, std=0.02):
    """Latent weights ~ N(0, std) as f32 [n, k]."""
    return (rng.standard_normal((n, k), dtype=np.float32) * np.float32(std)).astype(np.float32)


def synth_activations(rng, m, k, outliers=False):
    """Activations ~ N(0, 1) as f32 [m, k]; with outliers=True, 1 % of the entries are scaled x20."""
    x = rng.standard_normal((m, k), dtype=np.float32)
    if outliers:
        mask = rng.random((m, k)) < 0.01
        x = np.where(mask, x * np.float32(20.0), x).astype(np.float32)
    return x


def rel_err(a, b):
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    denom = np.maximum(np.abs(b), 1e-30)
    return float(np.max(np.abs(a - b) / denom)) if a.size else 0.0
