"""``hql.nn.Linear4bit`` as the reference's benchmark uses it (benchmark_linear4bit.py:495-508, 583)."""
import torch

import flh_amd as _pkg


class Linear4bit(torch.nn.Module):
    """Buffers ``weight`` [N, K/2] u8 (packed codes of the group-rotated weight) and ``weight_scales`` [N, K/g] fp16,
    filled by the caller from ``hql.had_and_quant``; ``forward`` takes fp16 activations."""

    def __init__(self, in_features, out_features, bias=False, dtype=torch.float16, group_size=128, device=None):
        super().__init__()
        if group_size not in (32, 64, 128) or in_features % group_size or in_features % 128:
            raise ValueError("group_size must be 32, 64 or 128 and divide in_features (a multiple of 128)")
        self.in_features, self.out_features, self.group_size = in_features, out_features, group_size
        self.register_buffer("weight", torch.zeros(out_features, in_features // 2, dtype=torch.uint8, device=device))
        self.register_buffer("weight_scales", torch.zeros(out_features, in_features // group_size, dtype=dtype, device=device))
        if bias:
            self.register_buffer("bias", torch.zeros(out_features, dtype=dtype, device=device))
        else:
            self.bias = None

    def forward(self, x):
        ops = _pkg._CUDA
        g = self.group_size
        lead = x.shape[:-1]
        rows = x.reshape(-1, g).contiguous()
        # activation scales stored divided by g: undoes the two unnormalised transforms (H x . H w = g . x w)
        if g == 128:
            q, s = ops.hadamard_and_quantize_i4(rows, scale_mul=1.0 / g)
        else:
            q, s = ops.hadamard_and_quantize_i4_gs(rows, g, scale_mul=1.0 / g)
        m = rows.size(0) * g // self.in_features
        y = ops.gemm_i4_dequant_o16_gs(q.view(m, self.in_features // 2), self.weight, s.view(m, -1), self.weight_scales, g)
        if self.bias is not None:
            y = y + self.bias
        return y.view(*lead, self.out_features)
