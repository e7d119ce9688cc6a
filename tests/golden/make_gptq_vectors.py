"""Write golden outputs of the reference's own GPTQ (flh/nn/gptq.py: FLHGPTQ.add_batch :127-144, fasterquant :146-237,
GPTQQuantizer :27-112) on the CPU, for the seeded inputs of gptq_inputs.py: a float32 nn.Linear(512, 64), 1500
calibration rows in three batches, activation order on / off, groups of 128 / one scale per row, clip ratio 1.0 / 0.9.

Runs in the authoring container only (the reference tree does not travel); ``gptq_vectors.npz`` next to this script is
data: a sample of the Hessian the reference accumulated, and per case `layer.weight` after `fasterquant`.
    python tests/golden/make_gptq_vectors.py
"""
import pathlib
import sys

import numpy as np
import torch

sys.path.insert(0, str(pathlib.Path(__file__).parent))
sys.path.insert(0, "/root/reference")
import gptq_inputs as G  # noqa: E402
import flh  # noqa: E402,F401  (degrades to _CUDA = None without a GPU)
from flh.nn.gptq import FLHGPTQ  # noqa: E402

OUT = pathlib.Path(__file__).with_name("gptq_vectors.npz")


def main():
    out = {}
    w = torch.from_numpy(G.weight())
    batches = [torch.from_numpy(b) for b in G.calibration_batches()]
    for label, group, actorder, clip in G.CASES:
        layer = torch.nn.Linear(G.COLS, G.ROWS, bias=False)
        layer.weight.data.copy_(w)
        gptq = FLHGPTQ(layer)
        for b in batches:
            gptq.add_batch(b, None, group_size=group)
        if f"hessian_g{group}_diag" not in out:         # (a sample of it: the diagonal, a corner block, one row)
            h = gptq.H.clone().numpy()
            out[f"hessian_g{group}_diag"] = np.diag(h).copy()
            out[f"hessian_g{group}_block"] = h[:48, :48].copy()
            out[f"hessian_g{group}_row300"] = h[300].copy()
        gptq.fasterquant(group_size=group, blocksize=128, percdamp=0.01, actorder=actorder, sym=True, bits=4, clip_ratio=clip)
        out[f"weight_{label}"] = layer.weight.data.clone().numpy()
        print(label, float(layer.weight.data.abs().max()))
    np.savez_compressed(OUT, **out)
    print("wrote", OUT, OUT.stat().st_size, "bytes")


if __name__ == "__main__":
    main()
