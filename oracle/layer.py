"""A W4A4 Llama decoder layer and decode step on the CPU (test infrastructure; see oracle/__init__.py): the
composition of the oracle's own pieces -- prologue.rmsnorm_f16 / silu_mul_f16, linear.rotate_and_quantize,
quant.act_quantizer_forward, gemm.gemm_i4_dequant -- with rotary embedding and attention evaluated in float64.

Reference lines followed
  * attention: flh/quantized_model/modeling_llama.py:374-470 -- quantiser, q / k / v projections from the same
    codes (:389-393), view as heads (:398-400), rotary embedding on q and k (:403-404), cache update (:406-424), causal
    softmax attention (flash-attn there: softmax(q k^T / sqrt(d)) v), quantiser, o_proj (:466-467);
  * MLP: :522-526 -- quantiser, act_fn(gate) * up, quantiser, down_proj;
  * layer and model: the residual structure of transformers' LlamaDecoderLayer that the reference inherits
    (x + attn(norm(x)); x + mlp(norm(x))), final norm and lm_head (:668-693);
  * rotary embedding: transformers' LlamaRotaryEmbedding / apply_rotary_pos_emb as the reference calls them (:403-404):
    inv_freq = theta^(-2i/d), angles = position * inv_freq duplicated over both halves, x cos + rotate_half(x) sin.
  * the two quantiser arrangements: "group" = ActQuantizer(use_hadamard=False) over groups of 128 (:322-325) with
    group-scaled weights; "token" = whole-row normalised Hadamard + one scale per token
    (benchmark/nn/benchmark_linear_flh.py:139-222, fake_quant/main.py:30-35 for the online rotation of down_proj).

Arithmetic outside the quantisers and GEMMs (RMSNorm statistics, rotary products, softmax, SiLU) is the executing
device's in the reference; here rotary embedding and attention run in float64 and are rounded to fp16 where the
reference holds fp16 tensors, so comparisons of whole layers with a device are by tolerance, while each quantiser and
each GEMM can be compared exactly when it is fed the device's own inputs (the `taps` of the device layer).

Pinning: everything quantised goes through functions pinned elsewhere in this package.  The float64 pieces are pinned
in tests/test_oracle_layer.py: attention with one key returns its value, uniform keys return the mean of the values,
a causal prefix is unaffected by later tokens, cached decoding equals prefill; rotary embedding is the identity at
position 0, preserves norms and makes q_m . k_n depend on m - n only.
"""
import numpy as np

from . import gemm, linear, prologue, quant
from .pack import pack_i4

_F16 = np.float16


def rotary_tables(positions, head_dim, theta=10000.0):
    """cos, sin [T, head_dim] as fp16 (float32 angles as the device computes them, then cos / sin, then fp16)."""
    inv = (1.0 / (np.float32(theta) ** (np.arange(0, head_dim, 2, dtype=np.float32) / np.float32(head_dim)))).astype(np.float32)
    ang = np.asarray(positions, dtype=np.float32)[:, None] * inv[None, :]
    ang = np.concatenate((ang, ang), axis=-1)
    return np.cos(ang.astype(np.float64)).astype(_F16), np.sin(ang.astype(np.float64)).astype(_F16)


def rotate_half(x):
    h = x.shape[-1] // 2
    return np.concatenate((-x[..., h:], x[..., :h]), axis=-1)


def apply_rotary(x, cos, sin):
    """x [B, H, T, d] fp16; cos / sin [T, d] fp16 -> fp16.  Products and the sum in float64, rounded once (the device
    rounds each fp16 product and the sum: at most two fp16 ulps apart)."""
    x64 = x.astype(np.float64)
    return (x64 * cos.astype(np.float64) + rotate_half(x64) * sin.astype(np.float64)).astype(_F16)


def attention_f64(q, k, v, past):
    """softmax(q k^T / sqrt(d)) v in float64.  q [B, H, T, d], k / v [B, Hkv, past + T, d] fp16; query t sees keys
    [0, past + t].  Grouped queries: head h uses key / value head h // (H / Hkv).  Returns fp16 [B, H, T, d]."""
    b, h, t, d = q.shape
    hkv = k.shape[1]
    rep = h // hkv
    k64 = np.repeat(k.astype(np.float64), rep, axis=1)
    v64 = np.repeat(v.astype(np.float64), rep, axis=1)
    scores = q.astype(np.float64) @ k64.transpose(0, 1, 3, 2) / np.sqrt(np.float64(d))
    n = k.shape[2]
    visible = np.arange(n)[None, :] <= (past + np.arange(t))[:, None]
    scores = np.where(visible[None, None], scores, -np.inf)
    scores -= scores.max(-1, keepdims=True)
    p = np.exp(scores)
    p /= p.sum(-1, keepdims=True)
    return (p @ v64).astype(_F16)


class LayerWeights:
    """Packed codes and scales of the seven linears (as the device layer holds them) and the two norm weights."""

    def __init__(self, packed, scales, norms, num_heads, num_kv_heads, eps=1e-5, activation="token", weight_group=128,
                 hadamard_mode="f32"):
        self.packed, self.scales, self.norms = packed, scales, norms
        self.num_heads, self.num_kv_heads, self.eps = num_heads, num_kv_heads, eps
        self.activation, self.weight_group, self.hadamard_mode = activation, weight_group, hadamard_mode


def quantise(w, x, norm_weight=None):
    """The quantiser in front of a linear: optional RMSNorm, then per the layer's arrangement.  x fp16 [M, K] ->
    (packed codes, scales, the fp16 rows that were quantised)."""
    h = prologue.rmsnorm_f16(x, norm_weight, w.eps) if norm_weight is not None else x
    if w.activation == "token":
        q, s, _ = linear.rotate_and_quantize(h, w.hadamard_mode)
        return q, s, h
    s, codes = quant.act_quantizer_forward(h, 128, False)
    return pack_i4(codes), s, h


def project(w, name, q, s):
    d, _ = gemm.gemm_i4_dequant(q, w.packed[name], s, w.scales[name], group=w.weight_group)
    return d


def decoder_layer(w, x, cos, sin, kv_cache=None, taps=None):
    """x fp16 [B, T, hidden]; cos / sin fp16 [T, head_dim] of the new positions; kv_cache: None or (keys, values)
    fp16 [B, Hkv, past, d].  Returns (y fp16 [B, T, hidden], (keys, values)).  `taps` (a dict) receives every stage."""
    taps = taps if taps is not None else {}
    b, t, hidden = x.shape
    hd = hidden // w.num_heads
    rows = x.reshape(b * t, hidden)
    q, s, _ = quantise(w, rows, w.norms["input_layernorm"])
    taps["attn_in.codes"], taps["attn_in.scales"] = q, s
    heads = {}
    for name, nh in (("q_proj", w.num_heads), ("k_proj", w.num_kv_heads), ("v_proj", w.num_kv_heads)):
        taps[name] = project(w, name, q, s)
        heads[name] = taps[name].reshape(b, t, nh, hd).transpose(0, 2, 1, 3)
    qs, ks, vs = apply_rotary(heads["q_proj"], cos, sin), apply_rotary(heads["k_proj"], cos, sin), heads["v_proj"]
    if kv_cache is not None:
        ks, vs = np.concatenate((kv_cache[0], ks), axis=2), np.concatenate((kv_cache[1], vs), axis=2)
    past = ks.shape[2] - t
    att = attention_f64(qs, ks, vs, past).transpose(0, 2, 1, 3).reshape(b * t, hidden)
    taps["attn_out.input"] = att
    q, s, _ = quantise(w, att)
    taps["attn_out.codes"], taps["attn_out.scales"] = q, s
    taps["o_proj"] = project(w, "o_proj", q, s)
    rows = (rows.astype(np.float32) + taps["o_proj"].astype(np.float32)).astype(_F16)       # fp16 residual add
    q, s, _ = quantise(w, rows, w.norms["post_attention_layernorm"])
    taps["mlp_in.codes"], taps["mlp_in.scales"] = q, s
    taps["gate_proj"], taps["up_proj"] = project(w, "gate_proj", q, s), project(w, "up_proj", q, s)
    mid = prologue.silu_mul_f16(taps["gate_proj"], taps["up_proj"])
    taps["mlp_mid.input"] = mid
    q, s, _ = quantise(w, mid)
    taps["mlp_mid.codes"], taps["mlp_mid.scales"] = q, s
    taps["down_proj"] = project(w, "down_proj", q, s)
    y = (rows.astype(np.float32) + taps["down_proj"].astype(np.float32)).astype(_F16)
    return y.reshape(b, t, hidden), (ks, vs)


def model_step(layers, x, positions, head_dim, theta, caches=None, final_norm=None, lm_head=None, eps=1e-5):
    """x fp16 [B, T, hidden] (the embedded tokens) through `layers` (LayerWeights), the final RMSNorm and the fp16
    head (float64 products rounded to fp16).  caches: None or a list of (keys, values) per layer.
    Returns (hidden or logits fp16, new caches)."""
    cos, sin = rotary_tables(positions, head_dim, theta)
    out_caches = []
    for i, w in enumerate(layers):
        x, c = decoder_layer(w, x, cos, sin, caches[i] if caches is not None else None)
        out_caches.append(c)
    if final_norm is not None:
        x = prologue.rmsnorm_f16(x, final_norm, eps)
    if lm_head is not None:
        x = (x.astype(np.float64) @ lm_head.astype(np.float64).T).astype(_F16)
    return x, out_caches
