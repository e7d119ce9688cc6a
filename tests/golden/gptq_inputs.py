"""Seeded inputs of the GPTQ fixtures (shared by the script that wrote them and the tests that read them): a float32
weight matrix [64, 512] and 1500 correlated calibration rows with a few loud channels, in three batches."""
import numpy as np

ROWS, COLS, SAMPLES = 64, 512, 1500
# (label, group_size, actorder, clip_ratio)
CASES = [(f"g{g}_{'act' if a else 'seq'}_clip{str(c).replace('.', '')}", g, a, c)
         for g in (128, -1) for a in (False, True) for c in (1.0, 0.9)]


def weight():
    rng = np.random.default_rng(20240611)
    return (rng.standard_normal((ROWS, COLS)) / np.sqrt(COLS)).astype(np.float32)


def calibration_batches():
    rng = np.random.default_rng(977)
    mix = rng.standard_normal((COLS, COLS)) / np.sqrt(COLS) + np.eye(COLS)   # correlated channels: the feedback matters
    x = rng.standard_normal((SAMPLES, COLS)) @ mix
    x[:, rng.permutation(COLS)[:5]] *= 20.0                                    # loud channels, as activations have them
    x = x.astype(np.float32)
    return [x[:500], x[500:1000], x[1000:]]
