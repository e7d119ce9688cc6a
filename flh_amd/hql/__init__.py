"""The legacy ``hql`` names that the reference's linear benchmark still imports
(benchmark_linear4bit.py:16-17, 495-508, 583):

    import hql; from hql.nn import Linear4bit
    layer = Linear4bit(in_features, out_features, bias=False, dtype=torch.float16, group_size=128).cuda()
    q, s = hql.had_and_quant(weight.view(-1, group_size))      # codes [R, g/2] u8, scales [R] fp16
    layer.weight.copy_(q.reshape(-1, in_features // 2)); layer.weight_scales.copy_(s.reshape(-1, in_features // g))
    y = layer(x)                                               # x fp16 [..., in_features]

The ``hql`` package itself is not part of the reference tree, so its arithmetic is taken from those call sites:
``had_and_quant`` is the group kernel of flh._CUDA.hadamard_and_quantize_i4[_gs] (unnormalised transform, raw scales),
and ``Linear4bit.forward`` quantises its fp16 input the same way and runs the group-scale GEMM.  Both operands then
carry an unnormalised Hadamard factor (H x . H w = g . x w per group), which the layer removes by storing the activation
scales divided by g, so that the output approximates ``x @ W.T`` as the benchmark's error check expects.  Parity with
the absent package is unpinned beyond that.  ``install_as_hql()`` registers the module under the name ``hql``.
"""
import sys

import flh_amd as _pkg

from . import nn  # noqa: F401


def had_and_quant(x):
    """x [R, g] fp16 with g in {32, 64, 128} -> (packed codes [R, g/2] u8, scales [R] fp16)."""
    g = x.size(-1)
    if g == 128:
        q, s = _pkg._CUDA.hadamard_and_quantize_i4(x.contiguous())
    else:
        q, s = _pkg._CUDA.hadamard_and_quantize_i4_gs(x.contiguous(), g)
    return q, s


def install_as_hql():
    me = sys.modules[__name__]
    sys.modules.setdefault("hql", me)
    sys.modules.setdefault("hql.nn", nn)
    return me
