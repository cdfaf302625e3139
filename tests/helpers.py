"""Shared input generators and comparison helpers for the test-suite."""
import json
import os

import numpy as np

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load_kat():
    with open(os.path.join(GOLDEN, "reference_kat.json")) as f:
        cases = json.load(f)["cases"]
    out = []
    for c in cases:
        out.append(
            dict(
                name=c["name"],
                rows=c["rows"],
                cols=c["cols"],
                dense=np.array(c["dense"], dtype=np.float16),
                values=np.array(c["values"], dtype=np.float16),
                deltas=np.array(c["deltas"], dtype=np.uint8),
                row_indices=np.array(c["row_indices"], dtype=np.int32),
            )
        )
    return out


def random_sparse(rng, rows, cols, density, scale=0.02, dist="normal"):
    """fp16 matrix with an unstructured Bernoulli mask."""
    if dist == "normal":
        m = (rng.standard_normal((rows, cols), dtype=np.float32) * scale).astype(np.float16)
    else:
        m = rng.random((rows, cols), dtype=np.float32).astype(np.float16)
    if density < 1.0:
        m[rng.random((rows, cols), dtype=np.float32) >= density] = 0
    return m


def row_pruned(rng, rows, cols, density, scale=0.02):
    """Per-row magnitude pruning: keep the round(density*cols) largest |w| of every row."""
    m = (rng.standard_normal((rows, cols), dtype=np.float32) * scale).astype(np.float16)
    keep = int(round(density * cols))
    if keep < cols:
        order = np.argsort(-np.abs(m.astype(np.float32)), axis=1, kind="stable")
        drop = order[:, keep:]
        np.put_along_axis(m, drop, np.float16(0), axis=1)
    return m


def skewed(rng, rows, cols, mean_density=0.3, alpha=1.5, lo=0.01, hi=0.95, zero_row_every=97, gap=40):
    """Per-row density from a power law clipped to [lo, hi] and rescaled to the wanted mean; some
    rows all zero; a run of `gap` zero columns in every row (forces padding entries)."""
    u = rng.random(rows)
    d = lo * (1.0 - u) ** (-1.0 / alpha)  # Pareto(alpha) scaled to start at lo
    d = np.clip(d, lo, hi)
    for _ in range(20):  # rescale towards the mean, re-clipping
        d = np.clip(d * (mean_density / d.mean()), lo, hi)
    m = (rng.standard_normal((rows, cols), dtype=np.float32) * 0.02).astype(np.float16)
    m[rng.random((rows, cols)) >= d[:, None]] = 0
    start = rng.integers(0, max(cols - gap, 1), size=rows)
    idx = start[:, None] + np.arange(gap)[None, :]
    np.put_along_axis(m, np.minimum(idx, cols - 1), np.float16(0), axis=1)
    m[::zero_row_every] = 0
    return m, d


def dense_reference(dense_f16, x_f16):
    """fp64 product of the fp16 data: what every implementation approximates."""
    return dense_f16.astype(np.float64) @ x_f16.astype(np.float64)


def assert_close_fp16(got_f16, want_f64, rel=1e-2, abs_=1e-3):
    """Bar stated for the path: |got - want| <= abs + rel * |want| elementwise."""
    got = np.asarray(got_f16, dtype=np.float64)
    err = np.abs(got - want_f64)
    bound = abs_ + rel * np.abs(want_f64)
    bad = err > bound
    assert not bad.any(), (
        f"{bad.sum()} of {bad.size} elements out of tolerance; worst err {err.max():.3e} "
        f"at {int(err.argmax())} (want {want_f64[err.argmax()]:.6e})"
    )
