"""One W4A4 Llama decoder layer on this library's kernels.

The data path of the reference's FLH_LlamaAttention / FLH_LlamaMLP inside a LlamaDecoderLayer
(flh/quantized_model/modeling_llama.py:374-470 attention with cache, :522-526 MLP; norms :655-656): every linear is
a LinearFLH fed by a quantiser,

    x -> RMSNorm -> quantiser -> q / k / v -> RoPE -> attention -> quantiser -> o_proj -> + x
      -> RMSNorm -> quantiser -> gate / up -> silu(gate) * up -> quantiser -> down_proj -> +

with torch's scaled_dot_product_attention in place of the flash-attn package.  The key / value cache is either a
plain tensor pair that grows by concatenation (prefill, tests) or one layer of a preallocated StaticKVCache
(decode steps that are captured into a graph).

`activation="group"` is the arrangement of the reference's quantised model: group quantisers of 128 without online
rotation (the rotations are folded into the weights and the embedding there) and group-scaled weights.
`fused=True` replaces "RMSNorm, quantiser" by one launch, the projections that share an input by one launch
(LinearFLH.forward_many) and "silu * up, quantiser" by one launch: the same bits as the module-by-module sequence,
which `fused=False` keeps for comparison.

`activation="token"` is the path's other configuration: every linear input is rotated as a whole row online
(normalised Hadamard of the hidden size; 172 x 64 resp. 28 x 512 for down_proj) and quantised with one scale per
token; the weights are rotated the same way offline and carry one scale per output channel
(`weight_group_size <= 0`, the arrangement of benchmark/nn/benchmark_linear_flh.py:139-222) or per group of 128
input channels (the Llama-3 configuration).  There `fused=True` means RMSNorm inside the rotation kernel, shared-input
launches and, for one or two tokens, the o_proj quantiser inside its GEMM.

`record`: when set to a dict, every quantiser's input / codes / scales and every linear's output of the next call
are stored in it (by stage name) -- the taps the parity tests compare with the CPU oracle stage by stage.
"""
import torch

from ..nn.fused import SiluMulQuant
from ..nn.linear import LinearFLH
from ..nn.normalization import RMSNorm
from ..nn.quantization import ActQuantizer


def rotary_tables(positions, head_dim, theta=10000.0, dtype=torch.float16):
    """cos / sin [T, head_dim] of Llama's rotary embedding for integer `positions` [T]."""
    inv = 1.0 / (theta ** (torch.arange(0, head_dim, 2, device=positions.device, dtype=torch.float32) / head_dim))
    ang = positions.to(torch.float32)[:, None] * inv[None, :]
    ang = torch.cat((ang, ang), dim=-1)
    return ang.cos().to(dtype), ang.sin().to(dtype)


def _decode_attention(q, k, v):
    """softmax(q k^T / sqrt(d)) v for ONE query position per sequence, as three batched matrix products' worth of stock
    tensor operations (the fused attention kernels are built for long query blocks and take 80 us for this shape):
    q [B, H, 1, d], k / v [B, Hkv, L, d] -> [B, H, 1, d]; query heads of one key / value head form the rows of a small
    matrix.  Scores and probabilities in float32."""
    b, h, _, d = q.shape
    hkv, n = k.size(1), k.size(2)
    qg = q.reshape(b * hkv, h // hkv, d)
    kt = k.reshape(b * hkv, n, d).transpose(1, 2)
    global _BMM_F32_OUT
    if _BMM_F32_OUT is None:                           # fp16 operands, float32 result, where this torch build has it
        try:
            torch.bmm(qg, kt, out_dtype=torch.float32)
            _BMM_F32_OUT = True
        except (TypeError, RuntimeError):
            _BMM_F32_OUT = False
    scores = torch.bmm(qg, kt, out_dtype=torch.float32) if _BMM_F32_OUT else torch.bmm(qg, kt).float()
    probs = torch.softmax(scores * (1.0 / d ** 0.5), dim=-1).to(q.dtype)
    return torch.bmm(probs, v.reshape(b * hkv, n, d)).reshape(b, h, 1, d)


_BMM_F32_OUT = None


def _rotate_half(x):
    half = x.size(-1) // 2
    return torch.cat((-x[..., half:], x[..., :half]), dim=-1)


class StaticKVCache:
    """Preallocated fp16 keys / values [layers][batch, kv_heads, max_len, head_dim].  `layer(i)` is what a decoder layer
    takes as `kv_cache`: new keys / values are written in place at `positions` and attention reads the first `kv_len`
    slots, causally for the last T of them.

    The contract between the two: a step over T new tokens runs with ``positions == arange(kv_len - T, kv_len)`` -- the
    new tokens take the last T of the slots attention reads.  `kv_len` is a host value and the causal structure is
    derived from it, not from `positions` (a device tensor the host does not read): other positions would let queries
    see slots that are not theirs to see, or leave the new keys outside what attention reads.  `advance(T)` sets both
    together.  For the same reason a captured graph serves ONE `kv_len` (it is a launch parameter, fixed at capture):
    replaying it after overwriting `positions` does not move the range attention reads -- capture one graph per length."""

    def __init__(self, layers, batch, kv_heads, max_len, head_dim, device, dtype=torch.float16, q_heads=None):
        self.keys = [torch.zeros(batch, kv_heads, max_len, head_dim, dtype=dtype, device=device) for _ in range(layers)]
        self.values = [torch.zeros_like(k) for k in self.keys]
        self.max_len = max_len
        self.kv_len = 0
        self._positions = torch.arange(max_len, dtype=torch.int64, device=device)   # advance() hands out views of it
        # the decode-attention kernel's scratch (partial results of the chunks), shared by the layers: they run in
        # order on one stream.  Owned here so that a captured graph finds it allocated.
        q_heads = q_heads or kv_heads * 8
        self.attention_workspace = torch.empty(batch * q_heads * ((max_len + 63) // 64) * (head_dim + 2) * 4,
                                               dtype=torch.uint8, device=device)

    class _Layer:
        def __init__(self, owner, index):
            self.owner, self.index = owner, index

        def rope_and_update(self, q, k, v, cos, sin, positions):
            """q [B, T, Hq, d] (rotated in place), k / v [B, T, Hkv, d] of the new tokens -> the first kv_len slots of
            this layer's keys / values, the new ones (keys rotated) written at `positions`."""
            keys, values = self.owner.keys[self.index], self.owner.values[self.index]
            _ops().rope_kv_cache_(q, k, v, cos, sin, positions, keys, values)
            n = self.owner.kv_len
            return keys[:, :, :n], values[:, :, :n]

        def tensors(self):
            return self.owner.keys[self.index], self.owner.values[self.index]

    def advance(self, t):
        """Make room for `t` new tokens behind what the cache holds: kv_len grows by t; returns the positions
        arange(kv_len - t, kv_len) (device int64 [t]) the step has to be run with."""
        if t < 1 or self.kv_len + t > self.max_len:
            raise ValueError(f"cannot advance a cache of {self.max_len} slots holding {self.kv_len} by {t}")
        self.kv_len += t
        return self._positions[self.kv_len - t:self.kv_len]

    def layer(self, index):
        return StaticKVCache._Layer(self, index)


class W4A4DecoderLayer(torch.nn.Module):
    PROJECTIONS = ("q_proj", "k_proj", "v_proj", "o_proj", "gate_proj", "up_proj", "down_proj")

    def __init__(self, hidden_size, num_heads, num_kv_heads, intermediate_size, eps=1e-5, act_group_size=128,
                 weight_group_size=128, fused=True, device="cpu", activation="group"):
        super().__init__()
        if activation not in ("group", "token"):
            raise ValueError("activation must be 'group' or 'token'")
        self.activation = activation
        if hidden_size % num_heads or num_heads % num_kv_heads:
            raise ValueError("hidden_size must divide into num_heads, num_heads into num_kv_heads")
        if act_group_size != 128:
            raise ValueError("ActQuantizer quantises groups of 128 (flh/nn/quantization.py:156-162)")
        self.hidden_size, self.num_heads, self.num_kv_heads = hidden_size, num_heads, num_kv_heads
        self.head_dim = hidden_size // num_heads
        self.intermediate_size, self.eps, self.fused = intermediate_size, eps, fused
        self.act_group_size = act_group_size
        self.weight_group_size = weight_group_size
        self.record = None
        # Token configuration, prefill-sized batches of the fused path: rotate rows of 4096 channels on the matrix cores
        # instead of with float32 butterflies (codes one step apart from the exactly rounded transform in fewer than 1e-4 of
        # the values -- closer to the float64 transform than the butterflies are -- for 5 us per launch at 4096 tokens).
        self.fast_rotation = False
        kv = num_kv_heads * self.head_dim
        shapes = {"q_proj": (hidden_size, hidden_size), "k_proj": (hidden_size, kv), "v_proj": (hidden_size, kv),
                  "o_proj": (hidden_size, hidden_size), "gate_proj": (hidden_size, intermediate_size),
                  "up_proj": (hidden_size, intermediate_size), "down_proj": (intermediate_size, hidden_size)}
        for name, (k, n) in shapes.items():
            g = weight_group_size if weight_group_size and weight_group_size > 0 else k
            setattr(self, name, LinearFLH(k, n, bias=False, device=device, in_group_size=act_group_size,
                                          group_size=g, no_hadamard=True))
        self.input_layernorm = RMSNorm(hidden_size, eps)
        self.post_attention_layernorm = RMSNorm(hidden_size, eps)

        def quantiser():
            return ActQuantizer(bits=4, group_size=act_group_size, sym=True, use_hadamard=False, packed_output=True)
        self.attn_quantizer1, self.attn_quantizer2 = quantiser(), quantiser()
        self.mlp_quantizer1, self.mlp_quantizer2 = quantiser(), quantiser()
        self._silu_mul_quant = SiluMulQuant(act_group_size)
        self._norm16 = {}     # fp16 copies of the norm weights for the fused kernels: name -> (version, tensor)

    @classmethod
    def from_float(cls, weights, num_heads, num_kv_heads, eps=1e-5, act_group_size=128, weight_group_size=None,
                   fused=True, activation="group", six_bit=False):
        """weights: fp16 tensors `q_proj` ... `down_proj` [N, K] (as nn.Linear stores them) and optionally
        `input_layernorm` / `post_attention_layernorm` [hidden]; quantised round-to-nearest ("group": as they are,
        "token": after the rotation of their input side).  weight_group_size: None = 128 for "group" and one scale
        per output channel for "token"; 128 with "token" is the Llama-3 arrangement; <= 0 one scale per channel.
        six_bit: LinearFLH.six_bit of the seven projections -- False (default), True or "auto" (group-scaled weights);
        anything but False costs a second copy of the weights (2.5 x the weight memory), built here."""
        hidden, inter = weights["q_proj"].size(1), weights["gate_proj"].size(0)
        device = weights["q_proj"].device
        if weight_group_size is None:
            weight_group_size = 128 if activation == "group" else 0
        layer = cls(hidden, num_heads, num_kv_heads, inter, eps, act_group_size, weight_group_size, fused, device,
                    activation)
        for name in cls.PROJECTIONS:
            w = weights[name]
            lin = getattr(layer, name)
            if activation == "token":
                # rows rotated by the same orthogonal transform as the activations
                g = lin.weight_group_size if lin.weight_group_size < w.size(1) else 0
                q, s = _ops().rotate_and_quantize_i4(w.to(torch.float16).contiguous(), hadamard="exact", scale_group=g)
                lin.w_packed.copy_(q.reshape(-1))
                lin.w_scale.copy_(s.reshape(lin.w_scale.shape))
                continue
            src = torch.nn.Linear(w.size(1), w.size(0), bias=False, device=device, dtype=w.dtype)
            src.weight.data.copy_(w)
            setattr(layer, name, LinearFLH.from_float(src, weight_group_size=weight_group_size,
                                                      in_group_size=act_group_size, no_hadamard=True))
        layer.set_six_bit(six_bit)
        for name in ("input_layernorm", "post_attention_layernorm"):
            norm = getattr(layer, name).to(device)
            if name in weights:
                norm.weight.data.copy_(weights[name].float())
        return layer

    # ------------------------------------------------------------------ pieces
    def _tap(self, name, value):
        if self.record is not None:
            self.record[name] = value.clone()      # a copy: q is rotated in place later on

    def _norm_weight16(self, name, norm):
        """The norm weight as the fused kernels take it (fp16; exact for weights that came from an fp16 checkpoint),
        converted once per version of the parameter."""
        w = norm.weight
        key = (w.data_ptr(), w._version)
        hit = self._norm16.get(name)
        if hit is None or hit[0] != key:
            hit = (key, w.detach().to(torch.float16).contiguous())
            self._norm16[name] = hit
        return hit[1]

    _F6_WIDTHS = (512, 1024, 2048, 4096, 8192, 11008, 14336)

    def set_six_bit(self, six_bit):
        """LinearFLH.six_bit of the seven projections (False, True, or "auto" / None), with the second encoding of the
        weights built at once where the setting can use it."""
        for name in self.PROJECTIONS:
            lin = getattr(self, name)
            lin.six_bit = None if six_bit == "auto" else six_bit
            if lin.w_packed.is_cuda:
                lin.prepare_six_bit()

    def _six_bit_for(self, consumers, n_rows, width):
        """Whether the quantiser in front of `consumers` should write the 6-bit operand format directly: every consumer
        would re-encode the nibbles for the 6-bit matrix instruction anyway."""
        return (bool(consumers) and self.activation == "token" and self.fused and self.record is None
                and width in self._F6_WIDTHS and all(l.wants_six_bit(n_rows) for l in consumers))

    def _rotation_mode(self, rows, k):
        """hadamard argument of the whole-row ops for `rows` rows of k channels."""
        fast = self.fast_rotation and self.fused and self.record is None and k == 4096 and rows > 64
        return "fast" if fast else True

    def _token_quant(self, stage, x, norm=None, norm_name=None, consumers=()):
        """Whole-row rotation + one scale per token (after RMSNorm when `norm` is given)."""
        rows = x.reshape(-1, x.size(-1)).contiguous()
        mode = self._rotation_mode(rows.size(0), rows.size(1))
        if self._six_bit_for(consumers, rows.size(0), rows.size(1)):
            if norm is not None:
                q, s = _ops().rotate_and_quantize_f6(rows, hadamard=mode, norm_weight=self._norm_weight16(norm_name, norm),
                                                     eps=norm.eps)
            else:
                q, s = _ops().rotate_and_quantize_f6(rows, hadamard=mode)
            return s.view(*x.shape[:-1], 1), None, q.view(*x.shape[:-1], -1)
        if norm is not None and self.fused:
            q, s = _ops().rmsnorm_rotate_and_quantize_i4(rows, self._norm_weight16(norm_name, norm), norm.eps, hadamard=mode)
        else:
            q, s = _ops().rotate_and_quantize_i4(norm(rows) if norm is not None else rows, hadamard=mode)
        self._tap(stage + ".input", rows)
        self._tap(stage + ".codes", q)
        self._tap(stage + ".scales", s)
        return s.view(*x.shape[:-1], 1), None, q.view(*x.shape[:-1], -1)

    def _norm_quant(self, stage, norm, norm_name, quantizer, x, consumers=()):
        if self.activation == "token":
            return self._token_quant(stage, x, norm, norm_name, consumers)
        if self.fused:
            q, s = _ops().rmsnorm_and_quantize_i4_gs(x.reshape(-1, x.size(-1)).contiguous(),
                                                     self._norm_weight16(norm_name, norm), norm.eps,
                                                     self.act_group_size, False)
            s, z, q = s.view(*x.shape[:-1], -1), None, q.view(*x.shape[:-1], -1)
        else:
            s, z, q = quantizer(norm(x))
        self._tap(stage + ".input", x.reshape(-1, x.size(-1)))
        self._tap(stage + ".codes", q.reshape(-1, q.size(-1)))
        self._tap(stage + ".scales", s.reshape(-1, s.size(-1)))
        return s, z, q

    def _residual_norm_quant(self, stage, norm, norm_name, quantizer, x, add, consumers=()):
        """(x + add, scales, zeros, codes): the residual addition (when `add` is given), the norm and the quantiser of
        the linears that follow (`consumers`) -- one launch where the whole-row path allows it, else the separate steps."""
        if add is None:
            return (x,) + tuple(self._norm_quant(stage, norm, norm_name, quantizer, x, consumers))
        k = x.size(-1)
        if k in (512, 1024, 2048, 4096, 8192) and self._six_bit_for(consumers, x.numel() // k, k):
            total, q, s = _ops().rotate_and_quantize_f6(
                x.reshape(-1, k).contiguous(), hadamard=self._rotation_mode(x.numel() // k, k),
                norm_weight=self._norm_weight16(norm_name, norm), eps=norm.eps, add=add.reshape(-1, k).contiguous())
            return total.view(x.shape), s.view(*x.shape[:-1], 1), None, q.view(*x.shape[:-1], -1)
        if self.activation == "token" and self.fused and self.record is None and k in (512, 1024, 2048, 4096, 8192):
            total, q, s = _ops().add_rmsnorm_rotate_and_quantize_i4(
                x.reshape(-1, k).contiguous(), add.reshape(-1, k).contiguous(), self._norm_weight16(norm_name, norm),
                norm.eps, hadamard=self._rotation_mode(x.numel() // k, k))
            return total.view(x.shape), s.view(*x.shape[:-1], 1), None, q.view(*x.shape[:-1], -1)
        x = x + add
        return (x,) + tuple(self._norm_quant(stage, norm, norm_name, quantizer, x, consumers))

    def _project(self, layers, q, s, z):
        if self.fused:
            return LinearFLH.forward_many(layers, q, s)
        return [layer(q, s, z, x_is_packed=True) for layer in layers]

    def attention(self, x, cos, sin, kv_cache=None, positions=None):
        """x [B, T, hidden] fp16 (already the residual stream); cos / sin [T, head_dim] of the T new positions;
        kv_cache: None, a pair (keys, values) [B, kv_heads, past, head_dim] that grows by concatenation, or one layer
        of a StaticKVCache together with `positions` (device int64 [T]: the slots the new tokens take, which must be
        arange(kv_len - T, kv_len) for the cache's kv_len, the number of slots attention reads -- see StaticKVCache).
        Causal over past + T positions."""
        _, y, cache = self._attention(x, None, cos, sin, kv_cache, positions, fold_residual=False)
        return y, cache

    def _attention(self, x, add, cos, sin, kv_cache=None, positions=None, fold_residual=True):
        """attention() on the residual stream x + add (add may be None): returns (that sum, the attention block's output,
        cache) -- or, when o_proj adds the residual in its epilogue (`fold_residual`, prefill sizes), (the stream after the
        block, None, cache)."""
        b, t, _ = x.shape
        if (self.activation == "token" and self.fused and self.record is None and b * t <= 2 and self.hidden_size == 4096
                and self._online_qkv_applies()):
            # decode: residual addition, norm, rotation, quantiser and the three projections in one launch
            layers = [self.q_proj, self.k_proj, self.v_proj]
            total, (qs, ks, vs) = _ops().rmsnorm_rotate_quantize_gemm_i4_multi(
                x.reshape(b * t, -1).contiguous(), None if add is None else add.reshape(b * t, -1).contiguous(),
                self._norm_weight16("input_layernorm", self.input_layernorm), self.input_layernorm.eps,
                [l.w_packed.view(l.out_features, l.in_features // 2) for l in layers],
                [l.w_scale.view(l.out_features, -1) for l in layers])
            if total is not None:
                x = total.view(x.shape)
        else:
            x, s, z, q = self._residual_norm_quant("attn_in", self.input_layernorm, "input_layernorm",
                                                   self.attn_quantizer1, x, add, (self.q_proj, self.k_proj, self.v_proj))
            mode = self._qkv_rope_applies(b * t, q, s, cos, kv_cache, positions)
            if mode:
                return self._attention_after_fused_qkv(x, q, s, cos, sin, kv_cache, positions, fold_residual, mode)
            qs, ks, vs = self._project([self.q_proj, self.k_proj, self.v_proj], q, s, z)
        self._tap("q_proj", qs), self._tap("k_proj", ks), self._tap("v_proj", vs)
        static = isinstance(kv_cache, StaticKVCache._Layer)
        out = None
        if (static and t == 1 and self.head_dim in (64, 128) and self.num_heads // self.num_kv_heads in (1, 2, 4, 8)
                and positions is not None):
            # one new token against the cache: rotary embedding, cache write and chunked attention in two launches
            keys, values = kv_cache.tensors()
            out = _ops().decode_attention_rope(qs.view(b, self.num_heads, self.head_dim),
                                               ks.view(b, self.num_kv_heads, self.head_dim),
                                               vs.view(b, self.num_kv_heads, self.head_dim), cos, sin, positions, keys,
                                               values, kv_cache.owner.kv_len,
                                               workspace=kv_cache.owner.attention_workspace)
            out = out.view(b, 1, self.hidden_size)
            cache = kv_cache
            past = kv_cache.owner.kv_len - 1
        elif static:
            # rotary embedding of q (in place) and k, and the new keys / values into their cache slots: one launch
            qs = qs.view(b, t, self.num_heads, self.head_dim)
            ks, vs = kv_cache.rope_and_update(qs, ks.view(b, t, self.num_kv_heads, self.head_dim),
                                              vs.view(b, t, self.num_kv_heads, self.head_dim), cos, sin, positions)
            cache = kv_cache
            if self._own_prefill_attention(t):
                out = _ops().prefill_attention(qs, *kv_cache.tensors(), kv_cache.owner.kv_len - t)
            qs = qs.transpose(1, 2)
        elif (self.fused and x.is_cuda and self.head_dim % 16 == 0 and cos.dtype == torch.float16
              and cos.shape == (t, self.head_dim)):
            # a growing pair of tensors as cache: the same rotary / cache-write launch on freshly allocated keys / values
            # (the bits of the tensor expression of the branch below, in one launch instead of a dozen)
            past = 0 if kv_cache is None else kv_cache[0].size(2)
            keys = torch.empty(b, self.num_kv_heads, past + t, self.head_dim, dtype=qs.dtype, device=x.device)
            values = torch.empty_like(keys)
            if past:
                keys[:, :, :past] = kv_cache[0]
                values[:, :, :past] = kv_cache[1]
            slots = torch.arange(past, past + t, device=x.device)
            qs = qs.view(b, t, self.num_heads, self.head_dim)
            _ops().rope_kv_cache_(qs, ks.view(b, t, self.num_kv_heads, self.head_dim),
                                  vs.view(b, t, self.num_kv_heads, self.head_dim), cos.contiguous(), sin.contiguous(),
                                  slots, keys, values)
            if self._own_prefill_attention(t):
                out = _ops().prefill_attention(qs, keys, values, past)
            qs = qs.transpose(1, 2)
            ks, vs = keys, values
            cache = (ks, vs)
        else:
            qs = qs.view(b, t, self.num_heads, self.head_dim).transpose(1, 2)
            ks = ks.view(b, t, self.num_kv_heads, self.head_dim).transpose(1, 2)
            vs = vs.view(b, t, self.num_kv_heads, self.head_dim).transpose(1, 2)
            qs = qs * cos + _rotate_half(qs) * sin
            ks = ks * cos + _rotate_half(ks) * sin
            if kv_cache is not None:
                ks, vs = torch.cat((kv_cache[0], ks), dim=2), torch.cat((kv_cache[1], vs), dim=2)
            cache = (ks, vs)
        gqa = self.num_heads != self.num_kv_heads
        if out is None:
            past = ks.size(2) - t
            if t == 1 and past > 0:
                out = _decode_attention(qs, ks, vs)           # one new token sees every cached position
            elif past == 0:
                out = torch.nn.functional.scaled_dot_product_attention(qs, ks, vs, is_causal=t > 1, enable_gqa=gqa)
            else:
                mask = torch.ones(t, past + t, dtype=torch.bool, device=x.device).tril(diagonal=past)
                out = torch.nn.functional.scaled_dot_product_attention(qs, ks, vs, attn_mask=mask, enable_gqa=gqa)
            out = out.transpose(1, 2).reshape(b, t, self.hidden_size).contiguous()
        if (self.activation == "token" and self.fused and self.record is None and b * t <= 2
                and self.hidden_size == 4096):
            # decode: the quantiser runs inside the GEMM's own launch (same bits as the two launches)
            return x, self.o_proj.forward_online(out, hadamard="exact"), cache
        return self._output_projection(x, out, cache, fold_residual)

    def _output_projection(self, x, out, cache, fold_residual):
        """quantiser + o_proj on the attention output `out` [B, T, hidden]; (stream, block output or None, cache) as
        _attention returns them."""
        s, z, q = (self._token_quant("attn_out", out, consumers=(self.o_proj,)) if self.activation == "token"
                   else self._group_quant("attn_out", self.attn_quantizer2, out))
        if fold_residual and self._residual_in_gemm(out.numel() // out.size(-1)):
            # prefill: the residual addition in o_proj's epilogue; nothing is left pending
            return self.o_proj(q, s, z, x_is_packed=True, residual=x), None, cache
        y = self.o_proj(q, s, z, x_is_packed=True)
        self._tap("o_proj", y)
        return x, y, cache

    def _own_prefill_attention(self, t):
        """Whether a block of t > 1 new tokens takes this library's causal-attention kernel (heads of 128 channels) instead
        of torch's fused attention."""
        return self.fused and self.record is None and t > 1 and self.head_dim == 128

    def _qkv_rope_applies(self, rows, codes, scales, cos, kv_cache, positions):
        """Whether q / k / v take the launch whose epilogue applies the rotary embedding and writes the cache -- the fused
        prefill path with heads of 128 channels and fp16 tables -- and on which matrix instruction: "i4" (nibble codes on
        the int8 kernel), "f6" (codes in the 6-bit format, or layers that would re-encode them) or None."""
        static = isinstance(kv_cache, StaticKVCache._Layer)
        if not (self.fused and self.record is None and rows > 64 and rows > codes.size(0) and self.head_dim == 128
                and codes.is_cuda and self._online_qkv_applies() and cos.dtype == torch.float16
                and tuple(cos.shape) == (rows // codes.size(0), 128) and (positions is not None if static else True)):
            return None
        if codes.size(-1) * 4 == self.hidden_size * 3:
            return "f6"
        if codes.size(-1) * 2 != self.hidden_size:
            return None
        layers = (self.q_proj, self.k_proj, self.v_proj)
        group = self.q_proj.weight_group_size if self.q_proj.weight_group_size > 0 else (self.q_proj.in_group_size or 128)
        six = all(l._six_bit_applies(codes.reshape(rows, -1), scales.reshape(rows, -1), l.w_scale.view(l.out_features, -1), group)
                  for l in layers)
        return "f6" if six else "i4"

    def _attention_after_fused_qkv(self, x, codes, scales, cos, sin, kv_cache, positions, fold_residual, mode):
        """The prefill attention block from the quantised input on: q / k / v, rotary embedding and cache write in one
        launch (the bits of the separate launches), torch's fused attention, then the output projection."""
        b, t, _ = x.shape
        layers = [self.q_proj, self.k_proj, self.v_proj]
        static = isinstance(kv_cache, StaticKVCache._Layer)
        if static:
            keys, values = kv_cache.tensors()
            slots, cache = positions, kv_cache
            past = None
        else:
            past = 0 if kv_cache is None else kv_cache[0].size(2)
            keys = torch.empty(b, self.num_kv_heads, past + t, self.head_dim, dtype=x.dtype, device=x.device)
            values = torch.empty_like(keys)
            if past:
                keys[:, :, :past] = kv_cache[0]
                values[:, :, :past] = kv_cache[1]
            slots = torch.arange(past, past + t, device=x.device)
            cache = (keys, values)
        group = self.q_proj.weight_group_size if self.q_proj.weight_group_size > 0 else (self.q_proj.in_group_size or 128)
        w_scales = [l.w_scale.view(l.out_features, -1) for l in layers]
        rows, a_rows = codes.reshape(b * t, -1), scales.reshape(b * t, -1)
        if mode == "f6":
            a6 = rows.contiguous() if rows.size(1) * 4 == self.hidden_size * 3 else _ops().encode_f6(rows.contiguous())
            qs = _ops().gemm_f6_qkv_rope(a6, a_rows.contiguous(), [l._six_bit_weights() for l in layers], w_scales,
                                         cos.contiguous(), sin.contiguous(), slots, keys, values, b)
        else:
            qs = _ops().gemm_i4_qkv_rope(rows, a_rows, [l.w_packed.view(l.out_features, l.in_features // 2) for l in layers],
                                         w_scales, cos.contiguous(), sin.contiguous(), slots, keys, values, b, group)
        if static:
            past = kv_cache.owner.kv_len - t
        # causal attention of the new block over the cache slots 0 .. past + t - 1, this library's kernel (heads of 128)
        out = _ops().prefill_attention(qs, keys, values, past)
        return self._output_projection(x, out, cache, fold_residual)

    def _residual_in_gemm(self, rows):
        """Whether o_proj / down_proj add the residual stream in their own epilogue: the fused prefill path of the group
        configuration, whose norm + quantiser launch has no addition of its own (measured at 2048 tokens: 728 against
        736 us per layer).  The token configuration keeps the addition inside its norm + rotation launch, which is cheaper
        than the extra read in the GEMM's epilogue burst (8 x 512 tokens: 888 against 910 us)."""
        return self.fused and self.record is None and rows > 64 and self.activation == "group"

    def _online_qkv_applies(self):
        """q / k / v in the layout the decode GEMM with its own norm + quantiser takes: no bias, one scale per channel or
        per group of 128, the same for all three."""
        cols = {l.w_scale.view(l.out_features, -1).size(1) for l in (self.q_proj, self.k_proj, self.v_proj)}
        if any(l.bias is not None for l in (self.q_proj, self.k_proj, self.v_proj)) or len(cols) != 1:
            return False
        c = cols.pop()
        return c == 1 or (c == self.hidden_size // 128 and self.q_proj.weight_group_size == 128)

    def _swiglu_gemm_applies(self):
        g = self.gate_proj
        cols = g.w_scale.view(g.out_features, -1).size(1)
        return g.bias is None and self.up_proj.bias is None and (cols == 1 or (g.weight_group_size == 128 and cols == g.in_features // 128))

    def _group_quant(self, stage, quantizer, x):
        s, z, q = quantizer(x)
        self._tap(stage + ".input", x.reshape(-1, x.size(-1)))
        self._tap(stage + ".codes", q.reshape(-1, q.size(-1)))
        self._tap(stage + ".scales", s.reshape(-1, s.size(-1)))
        return s, z, q

    def mlp(self, x):
        return self._mlp(x, None, fold_residual=False)[1]

    def _mlp(self, x, add, fold_residual=True):
        """mlp() on the residual stream x + add (add may be None); returns (that sum, the MLP's output) -- or (the stream
        after the block, None) when down_proj adds the residual in its epilogue (`fold_residual`, prefill sizes)."""
        x, s, z, q = self._residual_norm_quant("mlp_in", self.post_attention_layernorm, "post_attention_layernorm",
                                               self.mlp_quantizer1, x, add, (self.gate_proj, self.up_proj))
        rows = q.numel() // q.size(-1)
        if (self.activation == "token" and self.fused and self.record is None and rows > 64
                and self._swiglu_gemm_applies()):
            # prefill: gate and up in one launch that stores silu(gate) * up only (no fp16 [M, I] round trips)
            s, z, q = self._token_quant("mlp_mid", LinearFLH.forward_swiglu(self.gate_proj, self.up_proj, q, s),
                                        consumers=(self.down_proj,))
            if fold_residual:
                return self.down_proj(q, s, z, x_is_packed=True, residual=x), None
            return x, self.down_proj(q, s, z, x_is_packed=True)
        gate, up = self._project([self.gate_proj, self.up_proj], q, s, z)
        self._tap("gate_proj", gate), self._tap("up_proj", up)
        if (self.activation == "token" and self.fused and self.record is None and rows <= 256
                and self.intermediate_size in (11008, 14336)):
            # decode: silu(gate) * up formed inside the rotation's launch, never stored
            q, s = _ops().silu_mul_rotate_and_quantize_i4(gate.reshape(rows, -1), up.reshape(rows, -1))
            s, z, q = s.view(*x.shape[:-1], 1), None, q.view(*x.shape[:-1], -1)
        elif self.activation == "token":
            # (the library's product kernel when fused, so that every fused path sees the same fp16 product)
            mid = _ops().silu_mul(gate, up) if self.fused else torch.nn.functional.silu(gate) * up
            s, z, q = self._token_quant("mlp_mid", mid, consumers=(self.down_proj,))
        elif self.fused and self.record is None:
            s, z, q = self._silu_mul_quant(gate, up)
        else:
            s, z, q = self._group_quant("mlp_mid", self.mlp_quantizer2, torch.nn.functional.silu(gate) * up)
        if fold_residual and self._residual_in_gemm(rows):
            return self.down_proj(q, s, z, x_is_packed=True, residual=x), None
        y = self.down_proj(q, s, z, x_is_packed=True)
        self._tap("down_proj", y)
        return x, y

    def forward(self, x, cos, sin, kv_cache=None, positions=None):
        x, pending, cache = self.forward_deferred(x, None, cos, sin, kv_cache, positions)
        return (x if pending is None else x + pending), cache

    def forward_deferred(self, x, pending, cos, sin, kv_cache=None, positions=None):
        """The layer on the residual stream x + pending, with its own last addition left to the caller: returns
        (stream, pending, cache) with the layer's output = stream + pending (pending None: nothing left to add).  A stack
        of layers passes the pair on, so that every residual addition runs inside another launch: for a few tokens that
        of the norm + quantiser that reads its result, at prefill sizes the epilogue of the GEMM that produces the
        addend."""
        x, attn, cache = self._attention(x, pending, cos, sin, kv_cache, positions)
        x, y = self._mlp(x, attn)
        return x, y, cache


def _ops():
    import flh_amd
    return flh_amd._CUDA
