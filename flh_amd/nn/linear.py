"""W4A4 linear layer (reference: flh/nn/linear.py).

Buffers keep the reference's names and layouts: ``w_packed`` uint8 flat [N*K/2] (low nibble
= even input channel), ``w_scale`` [N, K/group] (or [N, 1] when group_size <= 0),
``w_zero`` uint8 (always 0: symmetric), optional ``bias``.  ``forward`` is one call of the
int4 GEMM + dequant kernel.  Unlike the reference's forward (flh/nn/linear.py:125-133, which
never adds it) the bias is added when the layer has one.
"""
import torch

import flh_amd as _pkg
from . import quantization as _quant
from ..functional.quantization import unpack_i4


class LinearFLH(torch.nn.Module):
    def __init__(self, in_features, out_features, bias=False, dtype=torch.float16, device="cpu",
                 dual_hadamard=False, in_group_size=None, out_group_size=None, no_hadamard=False, group_size=128):
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.dual_hadamard = dual_hadamard
        self.in_group_size = in_group_size
        self.out_group_size = out_group_size
        self.weight_group_size = group_size
        self.no_hadamard = no_hadamard
        n_groups = -(-in_features // group_size) if group_size > 0 else 1
        self.register_buffer("w_packed", torch.zeros((out_features * in_features + 1) // 2, dtype=torch.uint8, device=device))
        self.register_buffer("w_scale", torch.zeros(out_features, n_groups, dtype=dtype, device=device))
        self.register_buffer("w_zero", torch.zeros(out_features, n_groups, dtype=torch.uint8, device=device))
        if bias:
            self.register_buffer("bias", torch.zeros(out_features, dtype=dtype, device=device))
        else:
            self.bias = None
        # Opt-in (extension): run prefill-sized calls on the 6-bit matrix instruction (same bits, no unpack in the loop).
        # The layer then holds its weights a second time, re-encoded at 6 bits per code: 0.75 byte per weight on top of the
        # 0.5 of `w_packed`, i.e. 2.5 x the weight memory.  False (default): never.  True: every call of at least
        # `six_bit_min_rows` rows.  "auto" (or None): where it is faster even with the pass that re-encodes the activations
        # -- weights with a scale per group of 128.  `prepare_six_bit()` builds the second encoding at once (a loader calls
        # it); otherwise it is built on first use.  It is rebuilt whenever `w_packed` has been written to or replaced
        # (in-place copies, load_state_dict, .to(device)): keyed on the buffer's storage address and version counter.
        self.six_bit = False
        self.six_bit_min_rows = 256
        self._w6 = None
        self._w6_key = None

    def drop_six_bit_weights(self):
        self._w6 = self._w6_key = None

    def prepare_six_bit(self):
        """Build the 6-bit encoding of the weights now if this layer's setting can make use of it (at load time, rather
        than inside the first long call)."""
        if self.wants_six_bit(self.six_bit_min_rows):
            self._six_bit_weights()

    def _six_bit_weights(self):
        key = (self.w_packed.data_ptr(), self.w_packed._version, self.w_packed.device)
        if self._w6 is None or self._w6_key != key:
            self._w6 = _pkg._CUDA.encode_f6(self.w_packed.view(self.out_features, self.in_features // 2))
            self._w6_key = key
        return self._w6

    def wants_six_bit(self, n_rows):
        """Whether a call with `n_rows` per-token-quantised rows takes the 6-bit matrix instruction (a producer can then
        write the activations in that format directly, rotate_and_quantize_f6)."""
        if self.six_bit is False or n_rows < self.six_bit_min_rows or self.in_features % 128 or not self.w_packed.is_cuda:
            return False
        cols = self.w_scale.view(self.out_features, -1).size(1)
        if cols == 1:
            return self.six_bit is True
        return cols == self.in_features // 128 and self.weight_group_size == 128

    def _six_bit_applies(self, rows, a_scale, w_scale, group):
        if self.six_bit is False or not (rows.is_cuda and rows.size(0) >= self.six_bit_min_rows
                                         and self.in_features % 128 == 0):
            return False
        per_row = a_scale.size(1) == 1 and w_scale.size(1) == 1
        grouped = group == 128 and w_scale.size(1) == self.in_features // 128 and a_scale.size(1) in (1, w_scale.size(1))
        return grouped or (per_row and self.six_bit is True)

    # ------------------------------------------------------------------ kernels
    def forward(self, x, a_scale=None, a_zero=None, x_is_packed=False, is_symmetric=None, residual=None):
        """x: packed int4 activations [..., K/2] uint8; a_scale [..., K/in_group] or [..., 1]
        fp16 (as returned by ActQuantizer).  Returns fp16 [..., N].  `residual` (extension; fp16 [..., N]): returns
        residual + forward(x, ...) from the same launch -- the layer output rounded to fp16 as always, then one fp16
        addition in the GEMM's epilogue instead of a separate pass over both tensors."""
        lead = x.shape[:-1]
        if residual is not None and self.bias is not None:
            return residual + self.forward(x, a_scale, a_zero, x_is_packed, is_symmetric)
        res = None if residual is None else residual.reshape(-1, self.out_features)
        rows = x.view(-1, x.size(-1))
        w_scale = self.w_scale.view(self.out_features, -1)
        group = self.weight_group_size if self.weight_group_size > 0 else (self.in_group_size or 128)
        a_rows = a_scale.reshape(rows.size(0), -1)
        encoded = rows.size(1) * 4 == self.in_features * 3      # activations already in the 6-bit format
        if encoded or self._six_bit_applies(rows, a_rows, w_scale, group):
            ops = _pkg._CUDA
            w6 = self._six_bit_weights()
            a6 = rows.contiguous() if encoded else ops.encode_f6(rows.contiguous())
            if encoded and not ((w_scale.size(1) == 1 and a_rows.size(1) == 1) or
                                (group == 128 and w_scale.size(1) == self.in_features // 128)):
                raise ValueError("6-bit activations need per-token x per-channel scales or group-of-128 weight scales")
            if res is not None:
                y = ops.gemm_f6_dequant_add(a6, w6, a_rows.contiguous(), w_scale, res.contiguous())
            elif w_scale.size(1) == 1:
                y = ops.gemm_f6_dequant_o16(a6, w6, a_rows.contiguous(), w_scale)
            else:
                y = ops.gemm_f6_dequant_o16_gs(a6, w6, a_rows.contiguous(), w_scale)
            if self.bias is not None:
                y = y + self.bias
            return y.view(*lead, self.out_features)
        if res is not None:
            y = _pkg._CUDA.gemm_i4_dequant_add(rows, self.w_packed.view(self.out_features, self.in_features // 2),
                                               a_rows, w_scale, res.contiguous(), group)
            return y.view(*lead, self.out_features)
        y = _pkg._CUDA.gemm_i4_dequant(rows, self.w_packed.view(self.out_features, self.in_features // 2),
                                       a_scale.reshape(rows.size(0), -1), w_scale, group)
        if self.bias is not None:
            y = y + self.bias
        return y.view(*lead, self.out_features)

    @staticmethod
    def forward_many(layers, x, a_scale):
        """[layer(x, a_scale, x_is_packed=True) for layer in layers] in one GEMM launch: for projections that share
        their quantised input (q / k / v, gate / up; at most four), each with its own weights where they are.
        Same bits as the separate calls."""
        first = layers[0]
        lead = x.shape[:-1]
        rows = x.view(-1, x.size(-1))
        group = first.weight_group_size if first.weight_group_size > 0 else (first.in_group_size or 128)
        for layer in layers:
            if layer.in_features != first.in_features or layer.w_scale.shape[1:] != first.w_scale.shape[1:]:
                raise ValueError("forward_many: the layers must share in_features and the weight-scale layout")
        ops = _pkg._CUDA
        a_rows = a_scale.reshape(rows.size(0), -1)
        w_scales = [l.w_scale.view(l.out_features, -1) for l in layers]
        encoded = rows.size(1) * 4 == first.in_features * 3      # activations already in the 6-bit format
        if encoded or all(l._six_bit_applies(rows, a_rows, ws, group) for l, ws in zip(layers, w_scales)):
            # every layer opted into the 6-bit matrix instruction: one launch there as well
            a6 = rows.contiguous() if encoded else ops.encode_f6(rows.contiguous())
            ys = ops.gemm_f6_dequant_multi(a6, [l._six_bit_weights() for l in layers], a_rows.contiguous(), w_scales)
        else:
            ys = ops.gemm_i4_dequant_multi(rows, [l.w_packed.view(l.out_features, l.in_features // 2) for l in layers],
                                           a_rows, w_scales, group)
        return [(y if l.bias is None else y + l.bias).view(*lead, l.out_features) for y, l in zip(ys, layers)]

    @staticmethod
    def forward_swiglu(gate_layer, up_layer, x, a_scale):
        """act_fn(gate_layer(x)) * up_layer(x) of a SwiGLU MLP (flh/quantized_model/modeling_llama.py:522-526) in one
        GEMM launch that stores only the product: x packed codes [..., K/2], a_scale as for forward.  The two
        projections are rounded to fp16 as their own calls would store them, then combined as torch's fp16 silu and
        multiply do (the device's exponential: the fp16 result can differ from torch's in its last bit in a few values
        per thousand)."""
        if (gate_layer.in_features != up_layer.in_features or gate_layer.out_features != up_layer.out_features
                or gate_layer.w_scale.shape != up_layer.w_scale.shape):
            raise ValueError("forward_swiglu: gate and up must have the same shape and weight-scale layout")
        if gate_layer.bias is not None or up_layer.bias is not None:
            raise ValueError("forward_swiglu: layers with a bias take the separate calls")
        lead = x.shape[:-1]
        rows = x.view(-1, x.size(-1))
        n, k = gate_layer.out_features, gate_layer.in_features
        group = gate_layer.weight_group_size if gate_layer.weight_group_size > 0 else (gate_layer.in_group_size or 128)
        a_rows = a_scale.reshape(rows.size(0), -1)
        encoded = rows.size(1) * 4 == k * 3                     # activations already in the 6-bit format
        six = [l._six_bit_applies(rows, a_rows, l.w_scale.view(n, -1), group) for l in (gate_layer, up_layer)]
        if encoded or all(six):
            ops = _pkg._CUDA
            a6 = rows.contiguous() if encoded else ops.encode_f6(rows.contiguous())
            y = ops.gemm_f6_swiglu(a6, gate_layer._six_bit_weights(), up_layer._six_bit_weights(), a_rows.contiguous(),
                                   gate_layer.w_scale.view(n, -1), up_layer.w_scale.view(n, -1))
            return y.view(*lead, n)
        y = _pkg._CUDA.gemm_i4_swiglu(rows, gate_layer.w_packed.view(n, k // 2), up_layer.w_packed.view(n, k // 2),
                                      a_scale.reshape(rows.size(0), -1), gate_layer.w_scale.view(n, -1),
                                      up_layer.w_scale.view(n, -1), group)
        return y.view(*lead, n)

    def forward_online(self, x, hadamard=True):
        """fp16 activations [..., K] -> fp16 [..., N] with the activation side done here: whole-row rotation
        (`hadamard`: as in rotate_and_quantize_i4), one symmetric int4 scale per token, then the GEMM -- the
        online-Hadamard linear of the reference's benchmarks (benchmark/nn/benchmark_linear_flh.py:139-222), which
        has no module of its own there.  One or two tokens of K = 4096 with the bit-exact rotation take the
        single-launch decode path; the outputs are the same bits either way."""
        ops = _pkg._CUDA
        lead = x.shape[:-1]
        rows = x.reshape(-1, x.size(-1)).contiguous()
        w = self.w_packed.view(self.out_features, self.in_features // 2)
        w_scale = self.w_scale.view(self.out_features, -1)
        group = self.weight_group_size if self.weight_group_size > 0 else (self.in_group_size or 128)
        fusable = (0 < rows.size(0) <= 2 and self.in_features == 4096 and hadamard in (True, "exact")
                   and (w_scale.size(1) == 1 or (group == 128 and w_scale.size(1) == 32)))
        if fusable:
            y = ops.rotate_quantize_gemm_i4(rows, w, w_scale)
        else:
            q, s = ops.rotate_and_quantize_i4(rows, hadamard=hadamard)
            y = ops.gemm_i4_dequant(q, w, s, w_scale, group)
        if self.bias is not None:
            y = y + self.bias
        return y.view(*lead, self.out_features)

    # ------------------------------------------------------------------ torch arithmetic
    def _unpack_weights(self):
        """Dequantised weight [N, K] in the scale's dtype (flh/nn/linear.py:37-86)."""
        n, k = self.out_features, self.in_features
        w_int = unpack_i4(self.w_packed[: n * k // 2].view(n, k // 2)).float()
        g = self.weight_group_size
        if g > 0:
            wg = w_int.view(n, k // g, g) - self.w_zero.float().unsqueeze(-1)
            return (wg * self.w_scale.unsqueeze(-1)).view(n, k).to(self.w_scale.dtype)
        return ((w_int - self.w_zero.float()) * self.w_scale).to(self.w_scale.dtype)

    def _unpack_activation_4bit(self, x_packed, a_scale, a_zero, is_symmetric=None):
        """Packed codes -> dequantised float activations (flh/nn/linear.py:287-364)."""
        if is_symmetric is None:
            is_symmetric = not (a_zero is not None and torch.any(a_zero != 0))
        if is_symmetric:
            x_int = unpack_i4(x_packed).float()
        else:
            x_int = torch.stack((x_packed & 0x0F, x_packed >> 4), dim=-1).reshape(*x_packed.shape[:-1], -1).float()
        if a_scale is None:
            return x_int
        zp = a_zero if a_zero is not None else 0
        if self.in_group_size and self.in_group_size > 0 and a_scale.shape[-1] != 1:
            g = self.in_group_size
            v = x_int.view(*x_int.shape[:-1], -1, g)
            if torch.is_tensor(zp):
                zp = zp.view(*v.shape[:-1], 1)
            return ((v - zp) * a_scale.view(*v.shape[:-1], 1)).view_as(x_int)
        return (x_int - zp) * a_scale

    def forward_torch(self, x, a_scale=None, a_zero=None, x_is_packed=False, is_symmetric=None):
        if x_is_packed:
            x = self._unpack_activation_4bit(x, a_scale, a_zero, is_symmetric)
        elif a_scale is not None:
            zp = a_zero if a_zero is not None else 0
            x = (x - zp) * a_scale
        weight = self._unpack_weights()
        return torch.nn.functional.linear(x.to(weight.dtype), weight, self.bias)

    def get_weight(self, dtype=None):
        w = self._unpack_weights()
        return w if dtype is None else w.to(dtype)

    # ------------------------------------------------------------------ weight preparation
    def _pack_weights(self, w_int, scale, zero):
        """Store codes [N, K] (values in [-8, 7]) and their scales (flh/nn/linear.py:88-123)."""
        self.w_scale.copy_(scale.reshape(self.w_scale.shape))
        self.w_zero.copy_(zero.reshape(self.w_zero.shape).clamp(0, 15).to(torch.uint8))
        q = torch.clamp(w_int.flatten(), -8, 7).to(torch.int16) & 0xF
        if q.numel() % 2:
            q = torch.cat((q, q.new_zeros(1)))
        q = q.view(-1, 2)
        self.w_packed.copy_((q[:, 0] | (q[:, 1] << 4)).to(torch.uint8))

    def _quantize_and_store(self, W, bits, group_size, sym, clip_ratio):
        # fp16 weights that already sit on the GPU take the HIP quantise-and-pack kernel (same scales and
        # codes as the tensor arithmetic below: scale = fp16(max|w| / 7) per group or per row, codes =
        # clamp(rint(w / scale)); an all-zero group gets scale 1 where that arithmetic yields NaN)
        k = W.shape[-1]
        g = group_size if group_size and group_size > 0 else 0
        if (W.is_cuda and W.dtype == torch.float16 and W.dim() == 2 and bits == 4 and sym and clip_ratio >= 1.0
                and k % 16 == 0 and (g == 0 or (k % g == 0 and g % 2 == 0)) and self.w_scale.numel() == W.shape[0] * (k // g if g else 1)):
            q, s = _pkg._CUDA.rotate_and_quantize_i4(W.contiguous(), hadamard=False, scale_group=g)
            self.w_packed.copy_(q.reshape(self.w_packed.shape))
            self.w_scale.copy_(s.reshape(self.w_scale.shape))
            self.w_zero.zero_()
            return
        wq = _quant.WeightQuantizer(bits=bits, group_size=group_size, sym=sym, channel_wise=(group_size == -1),
                                    use_hadamard=False, clip_ratio=clip_ratio)
        wq.calibrate(W)
        if bits < 16 and torch.isnan(wq.scale).any():
            print(f"WARNING: NaN detected in quantization scale for layer {self.out_features}x{self.in_features}")
            return
        scale, zp, w_int = wq.quantize(W)
        if scale.dim() == 1:  # per tensor
            scale = scale.expand(self.out_features, 1)
            zp = zp.expand(self.out_features, 1)
        self._pack_weights(w_int, scale, zp)

    def set_weight(self, weight):
        """Quantise a float weight [N, K] (RTN, symmetric 4 bit, this layer's group size)."""
        self._quantize_and_store(weight, 4, self.weight_group_size, True, 1.0)

    @staticmethod
    def from_float(module, weight_bits=4, weight_group_size=128, weight_sym=True, dual_hadamard=False,
                   in_group_size=None, out_group_size=None, clip_ratio=1.0, no_hadamard=False):
        """Build from an nn.Linear (flh/nn/linear.py:190-285): optionally rotate the weight by
        the (grouped) normalised Hadamard matrix on the input side -- and on the output side,
        with the bias, when dual_hadamard -- then quantise and pack."""
        layer = LinearFLH(module.in_features, module.out_features, bias=module.bias is not None,
                          dtype=module.weight.dtype, device=module.weight.device, dual_hadamard=dual_hadamard,
                          in_group_size=in_group_size, out_group_size=out_group_size, group_size=weight_group_size)
        W = module.weight.data.clone()
        if layer.bias is not None:
            layer.bias.copy_(module.bias.data)
        if not no_hadamard:
            rot = _quant.fast_hadamard_transform
            if dual_hadamard:
                W = rot(W, group_size=in_group_size, use_cuda=False)
                W = rot(W.T, group_size=out_group_size, use_cuda=False).T
                if layer.bias is not None:
                    layer.bias.copy_(rot(layer.bias.unsqueeze(0), group_size=out_group_size).squeeze(0))
            else:
                W = rot(W, group_size=in_group_size)
        if torch.isnan(W).any():
            print(f"WARNING: NaN detected in weights after Hadamard for layer {module.out_features}x{module.in_features}")
            return layer
        layer._quantize_and_store(W.contiguous(), weight_bits, weight_group_size, weight_sym, clip_ratio)
        return layer
