"""GPTQ in the Hadamard-rotated basis on the CPU (test infrastructure; see oracle/__init__.py).

Reference lines followed: flh/nn/gptq.py:127-144 (`add_batch`: H = running mean of 2 x x^T over the rotated inputs),
:146-237 (`fasterquant`: rotation of the weights :160-164, dead columns :170-172, clipping and the per-group grids
fixed beforehand :176-183, activation order :185-189, damping :192-194, error feedback column by column :201-231),
:27-112 (`GPTQQuantizer`: symmetric grid scale = max|w| clamp(1e-5) / maxq, q = clamp(round(w / scale), -maxq - 1, maxq)).

The reference evaluates the feedback through the upper Cholesky factor of H^-1, block by block.  Here it is written in
the form the algorithm is derived in (optimal brain quantisation): after column i has been rounded, the remaining
columns move by  -(w_i - q_i) / [H^-1]_ii * [H^-1]_i,:  and column i is eliminated from H^-1 by one step of Gaussian
elimination -- no Cholesky factor, no blocks, float64.  Both are the same function of (W, H); this one shares no
formula with the implementation it checks.

Pinning (tests/test_oracle_gptq.py): with a diagonal H nothing is fed back and the result is round-to-nearest on the
same grids (closed form); the feedback leaves the layer output on the calibration inputs closer to the float layer's
than round-to-nearest does; the Hessian of `hessian` equals 2/N X^T X however the rows are split into batches; and the
reference's own `FLHGPTQ` (run on the CPU by tests/golden/make_gptq_vectors.py) on a seeded 64 x 512 layer with 1500
calibration rows -- groups of 128 / one scale per row, activation order on / off, clip ratio 1.0 / 0.9: the same
dequantised weights to float32 rounding in seven of the eight cases, and in the eighth in all rows but one (a column on
a rounding boundary in float32 and not in float64 flips one code, and the feedback moves later codes of that row).
"""
import numpy as np

from . import hadamard


def rotate_rows(x, group_size=None):
    """fast_hadamard_transform(x.float(), group_size) on rows: normalised, float64 here."""
    return hadamard.had_transform(np.asarray(x, dtype=np.float64), group_size)


def hessian(batches, group_size=None):
    """The running mean `add_batch` accumulates, from a list of input arrays [..., columns]."""
    h, n = None, 0
    for inp in batches:
        rows = rotate_rows(np.asarray(inp, dtype=np.float64).reshape(-1, inp.shape[-1]), group_size)
        m = rows.shape[0]
        h = np.zeros((rows.shape[1],) * 2) if h is None else h * (n / (n + m))
        n += m
        x = np.sqrt(2.0 / n) * rows.T
        h = h + x @ x.T
    return h


def grid_scales(w, group_size, bits=4, clip_ratio=1.0):
    """Symmetric per-group (or per-row when group_size <= 0) scales of the clipped weights, [rows, groups]."""
    maxq = 2 ** (bits - 1) - 1
    rows, cols = w.shape
    g = group_size if group_size and group_size > 0 and cols % group_size == 0 else cols
    v = w.reshape(rows, cols // g, g)
    if clip_ratio < 1.0:
        bound = np.abs(v).max(axis=2, keepdims=True) * clip_ratio
        v = np.clip(v, -bound, bound)
    return np.maximum(np.abs(v).max(axis=2), 1e-5) / maxq, g


def quantise_column(w, scale, bits=4, clip_ratio=1.0):
    maxq = 2 ** (bits - 1) - 1
    if clip_ratio < 1.0:
        bound = scale * maxq * clip_ratio
        w = np.clip(w, -bound, bound)
    return scale * np.clip(np.rint(w / scale), -(maxq + 1), maxq)


def gptq(weight, h, group_size=128, bits=4, percdamp=0.01, actorder=False, clip_ratio=1.0, dual_hadamard=False):
    """weight [rows, cols] (unrotated), h [cols, cols] from `hessian` -> dequantised weights of the rotated basis."""
    w = rotate_rows(weight, group_size if group_size and group_size > 0 else None)
    if dual_hadamard:
        w = rotate_rows(w.T, group_size if group_size and group_size > 0 else None).T
    h = np.array(h, dtype=np.float64)
    cols = w.shape[1]
    dead = np.diag(h) == 0
    h[dead, dead] = 1
    w[:, dead] = 0
    if clip_ratio < 1.0:                       # the weights themselves are clipped once, the grids clip once more
        g = group_size if group_size and group_size > 0 and cols % group_size == 0 else cols
        v = w.reshape(w.shape[0], cols // g, g)
        bound = np.abs(v).max(axis=2, keepdims=True) * clip_ratio
        w = np.clip(v, -bound, bound).reshape(w.shape)
    scales, g = grid_scales(w, group_size, bits, clip_ratio)
    order = np.argsort(-np.diag(h), kind="stable") if actorder else np.arange(cols)
    w = w[:, order]
    h = h[order][:, order]
    h[np.arange(cols), np.arange(cols)] += percdamp * np.mean(np.diag(h))
    hinv = np.linalg.inv(h)
    q = np.zeros_like(w)
    for i in range(cols):
        q[:, i] = quantise_column(w[:, i], scales[:, order[i] // g], bits, clip_ratio)
        err = (w[:, i] - q[:, i]) / hinv[i, i]
        w[:, i + 1:] -= np.outer(err, hinv[i, i + 1:])
        hinv[i + 1:, i + 1:] -= np.outer(hinv[i + 1:, i], hinv[i, i + 1:]) / hinv[i, i]
    out = np.empty_like(q)
    out[:, order] = q
    return out
