"""Pins of the float64 pieces of oracle/layer.py (rotary embedding, attention, cache handling) and of the layer's
wiring, by properties the mathematics fixes -- not by retyping the formulas."""
import numpy as np

from oracle import layer as OL
from oracle import prologue
from oracle.pack import pack_i4


def rand16(rng, *shape):
    return rng.standard_normal(shape).astype(np.float16)


def test_attention_special_cases():
    rng = np.random.default_rng(0)
    q = rand16(rng, 2, 4, 1, 16)
    v1 = rand16(rng, 2, 2, 1, 16)
    # one visible key: the output is its value, whatever the scores (grouped queries: heads 0, 1 -> kv head 0)
    out = OL.attention_f64(q, rand16(rng, 2, 2, 1, 16), v1, past=0)
    assert np.array_equal(out, np.repeat(v1, 2, axis=1))
    # identical keys: uniform weights, the output is the mean of the values
    k = np.repeat(rand16(rng, 2, 2, 1, 16), 5, axis=2)
    v = rand16(rng, 2, 2, 5, 16)
    out = OL.attention_f64(q, k, v, past=4)
    want = np.repeat(v.astype(np.float64).mean(2, keepdims=True), 2, axis=1)
    assert np.allclose(out.astype(np.float64), want, atol=2e-3)
    # a dominant score picks its value: key 3 = 50 * q direction
    k = rand16(rng, 1, 1, 6, 16) * np.float16(0.01)
    qq = rand16(rng, 1, 1, 1, 16)
    k[0, 0, 3] = qq[0, 0, 0] * np.float16(8)
    v = rand16(rng, 1, 1, 6, 16)
    out = OL.attention_f64(qq, k, v, past=5)
    assert np.allclose(out[0, 0, 0].astype(np.float64), v[0, 0, 3].astype(np.float64), atol=2e-2)


def test_attention_is_causal_and_cache_equals_prefill():
    rng = np.random.default_rng(1)
    b, h, hkv, t, d = 2, 4, 2, 7, 8
    q, k, v = rand16(rng, b, h, t, d), rand16(rng, b, hkv, t, d), rand16(rng, b, hkv, t, d)
    full = OL.attention_f64(q, k, v, past=0)
    # prefix property: the first 4 outputs do not depend on tokens 4 ..
    k2, v2 = k.copy(), v.copy()
    k2[:, :, 4:] = rand16(rng, b, hkv, t - 4, d)
    v2[:, :, 4:] = rand16(rng, b, hkv, t - 4, d)
    assert np.array_equal(OL.attention_f64(q, k2, v2, past=0)[:, :, :4], full[:, :, :4])
    # one query at a time against the growing key set gives the same rows
    for i in range(t):
        step = OL.attention_f64(q[:, :, i:i + 1], k[:, :, :i + 1], v[:, :, :i + 1], past=i)
        assert np.array_equal(step[:, :, 0], full[:, :, i])


def test_rotary_embedding_properties():
    rng = np.random.default_rng(2)
    d = 32
    cos, sin = OL.rotary_tables(np.arange(40), d, theta=10000.0)
    x = rand16(rng, 1, 2, 40, d)
    y = OL.apply_rotary(x, cos, sin)
    assert np.array_equal(y[:, :, 0], x[:, :, 0])                      # position 0: identity
    nx = np.linalg.norm(x.astype(np.float64), axis=-1)
    ny = np.linalg.norm(y.astype(np.float64), axis=-1)
    assert np.allclose(nx, ny, rtol=2e-3)                              # a rotation: norms kept
    # q_m . k_n depends on m - n only: the same vectors placed at (m, n) and (m + 9, n + 9)
    qv, kv = rand16(rng, d), rand16(rng, d)
    xs = np.zeros((1, 1, 40, d), dtype=np.float16)

    def dot(m, n):
        a, b = xs.copy(), xs.copy()
        a[0, 0, m], b[0, 0, n] = qv, kv
        ra, rb = OL.apply_rotary(a, cos, sin), OL.apply_rotary(b, cos, sin)
        return float(ra[0, 0, m].astype(np.float64) @ rb[0, 0, n].astype(np.float64))
    assert abs(dot(5, 2) - dot(14, 11)) < 0.05 * abs(dot(5, 2)) + 0.05
    assert abs(dot(5, 2) - dot(2, 5)) > 1e-3                           # ... and on its sign
    # the pair structure: channel i rotates with channel i + d/2 by angle pos * theta^(-2i/d)
    e = np.zeros((1, 1, 40, d), dtype=np.float16)
    e[0, 0, :, 3] = 1
    r = OL.apply_rotary(e, cos, sin).astype(np.float64)
    ang = np.arange(40) * 10000.0 ** (-2 * 3 / d)
    assert np.allclose(r[0, 0, :, 3], np.cos(ang), atol=2e-3) and np.allclose(r[0, 0, :, 3 + d // 2], np.sin(ang), atol=2e-3)
    assert np.abs(np.delete(r[0, 0], [3, 3 + d // 2], axis=-1)).max() == 0


def tiny_layer(activation, weight_group, seed=3, hidden=256, heads=4, kv_heads=2, inter=512):
    """Exactly representable weights: every linear is s * (integer codes), so the float path below is exact."""
    rng = np.random.default_rng(seed)
    hd = hidden // heads
    dims = {"q_proj": (hidden, hidden), "k_proj": (kv_heads * hd, hidden), "v_proj": (kv_heads * hd, hidden),
            "o_proj": (hidden, hidden), "gate_proj": (inter, hidden), "up_proj": (inter, hidden), "down_proj": (hidden, inter)}
    codes = {n: rng.integers(-8, 8, size=s, dtype=np.int8) for n, s in dims.items()}
    scales = {n: np.full((s[0], 1 if weight_group <= 0 else s[1] // weight_group), 2.0 ** -7, dtype=np.float16)
              for n, s in dims.items()}
    norms = {"input_layernorm": np.ones(hidden, np.float16), "post_attention_layernorm": np.ones(hidden, np.float16)}
    w = OL.LayerWeights({n: pack_i4(c) for n, c in codes.items()}, scales, norms, heads, kv_heads, 1e-5, activation,
                        weight_group if weight_group > 0 else 128)
    return w, codes


def test_layer_wiring_against_a_float_evaluation():
    """The quantised layer against the same layer evaluated in float64 with the dequantised weights and unquantised
    activations: int4 activation noise only (a wrong scale, a dropped residual, a transposed head layout or a missing
    rotation on one side would be O(1))."""
    for activation, group in (("token", 0), ("token", 128), ("group", 128)):
        w, codes = tiny_layer(activation, group)
        rng = np.random.default_rng(4)
        b, t, hidden = 2, 6, 256
        x = rand16(rng, b, t, hidden)
        hd = hidden // w.num_heads
        cos, sin = OL.rotary_tables(np.arange(t), hd)
        taps = {}
        y, (ks, vs) = OL.decoder_layer(w, x, cos, sin, taps=taps)
        assert y.shape == x.shape and ks.shape == (b, 2, t, hd) and y.dtype == np.float16
        # float evaluation; in the token arrangement the stored weights act on rotated inputs: W_eff = W_stored . H / sqrt(K)
        from oracle import hadamard as H

        def eff(name):
            wf = codes[name].astype(np.float64) * 2.0 ** -7
            if activation == "token":
                k = wf.shape[1]
                wf = wf @ (H.hadamard_matrix(k).astype(np.float64) / np.sqrt(k))
            return wf
        rows = x.reshape(b * t, hidden).astype(np.float64)

        def norm(v):
            return v / np.sqrt((v * v).mean(-1, keepdims=True) + 1e-5)
        h = norm(rows)
        q = (h @ eff("q_proj").T).reshape(b, t, 4, hd).transpose(0, 2, 1, 3)
        k = (h @ eff("k_proj").T).reshape(b, t, 2, hd).transpose(0, 2, 1, 3)
        v = (h @ eff("v_proj").T).reshape(b, t, 2, hd).transpose(0, 2, 1, 3)
        c64, s64 = cos.astype(np.float64), sin.astype(np.float64)
        def swap(v):          # (x1, x2) -> (-x2, x1), written out independently of the oracle's helper
            return np.concatenate((-v[..., hd // 2:], v[..., :hd // 2]), axis=-1)
        q, k = q * c64 + swap(q) * s64, k * c64 + swap(k) * s64
        kk, vv = np.repeat(k, 2, 1), np.repeat(v, 2, 1)
        sc = q @ kk.transpose(0, 1, 3, 2) / np.sqrt(hd)
        sc = np.where(np.tril(np.ones((t, t), bool))[None, None], sc, -np.inf)
        p = np.exp(sc - sc.max(-1, keepdims=True))
        att = ((p / p.sum(-1, keepdims=True)) @ vv).transpose(0, 2, 1, 3).reshape(b * t, hidden)
        rows = rows + att @ eff("o_proj").T
        h = norm(rows)
        g, u = h @ eff("gate_proj").T, h @ eff("up_proj").T
        want = rows + (g / (1 + np.exp(-g)) * u) @ eff("down_proj").T
        upd = np.linalg.norm(want - x.reshape(b * t, hidden).astype(np.float64))
        err = np.linalg.norm(y.reshape(b * t, hidden).astype(np.float64) - want) / upd
        assert err < 0.25, (activation, group, err)


def test_cached_decoding_equals_prefill_in_the_oracle_layer():
    w, _ = tiny_layer("token", 128, seed=5)
    rng = np.random.default_rng(6)
    t, hidden, hd = 5, 256, 64
    x = rand16(rng, 1, t, hidden)
    cos, sin = OL.rotary_tables(np.arange(t), hd)
    full, _ = OL.decoder_layer(w, x, cos, sin)
    cache, outs = None, []
    for i in range(t):
        y, cache = OL.decoder_layer(w, x[:, i:i + 1], cos[i:i + 1], sin[i:i + 1], cache)
        outs.append(y)
    assert np.array_equal(np.concatenate(outs, axis=1), full)       # per-token quantisers: identical operands


def test_model_step_head_and_norm():
    w, _ = tiny_layer("token", 128, seed=7)
    rng = np.random.default_rng(8)
    x = rand16(rng, 2, 1, 256)
    head = rand16(rng, 50, 256)
    fn = (rng.uniform(0.5, 1.5, 256)).astype(np.float16)
    hid, caches = OL.model_step([w, w], x, np.array([0]), 64, 10000.0, final_norm=fn)
    logits, _ = OL.model_step([w, w], x, np.array([0]), 64, 10000.0, final_norm=fn, lm_head=head)
    assert len(caches) == 2 and caches[0][0].shape == (2, 2, 1, 64)
    assert np.array_equal(logits, (hid.astype(np.float64) @ head.astype(np.float64).T).astype(np.float16))
    y1, _ = OL.decoder_layer(w, x, *OL.rotary_tables(np.array([0]), 64))
    y2, _ = OL.decoder_layer(w, y1, *OL.rotary_tables(np.array([0]), 64))
    assert np.array_equal(hid, prologue.rmsnorm_f16(y2, fn, 1e-5))
