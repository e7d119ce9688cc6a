"""The W4A4 decoder layer built from this library's modules: the fused form against the module-by-module form
(bit-equal), prefill against token-by-token decoding with the key / value cache, and the whole layer against the
same layer in fp16 (a loose bound: int4 noise)."""
import pytest
import torch

from flh_amd.quantized_model import W4A4DecoderLayer, rotary_tables

pytestmark = pytest.mark.gpu


def make(hidden=512, heads=4, kv_heads=2, inter=1024, seed=0, fused=True, activation="group"):
    g = torch.Generator(device="cpu").manual_seed(seed)
    kv = hidden // heads * kv_heads
    shapes = {"q_proj": (hidden, hidden), "k_proj": (kv, hidden), "v_proj": (kv, hidden), "o_proj": (hidden, hidden),
              "gate_proj": (inter, hidden), "up_proj": (inter, hidden), "down_proj": (hidden, inter)}
    w = {n: (torch.randn(s, generator=g) / s[1] ** 0.5).half().cuda() for n, s in shapes.items()}
    w["input_layernorm"] = (torch.rand(hidden, generator=g) + 0.5).half().cuda()
    w["post_attention_layernorm"] = (torch.rand(hidden, generator=g) + 0.5).half().cuda()
    return w, W4A4DecoderLayer.from_float(w, heads, kv_heads, fused=fused, activation=activation)


def fp16_layer(w, x, cos, sin, heads, kv_heads, eps=1e-5):
    def norm(v, weight):
        f = v.float()
        return (f * torch.rsqrt(f.pow(2).mean(-1, keepdim=True) + eps) * weight.float()).half()

    def rot(v):
        h = v.size(-1) // 2
        return torch.cat((-v[..., h:], v[..., :h]), dim=-1)
    b, t, hidden = x.shape
    hd = hidden // heads
    h = norm(x, w["input_layernorm"])
    q = (h @ w["q_proj"].T).view(b, t, heads, hd).transpose(1, 2)
    k = (h @ w["k_proj"].T).view(b, t, kv_heads, hd).transpose(1, 2)
    v = (h @ w["v_proj"].T).view(b, t, kv_heads, hd).transpose(1, 2)
    q, k = q * cos + rot(q) * sin, k * cos + rot(k) * sin
    k, v = k.repeat_interleave(heads // kv_heads, 1), v.repeat_interleave(heads // kv_heads, 1)
    a = torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True).transpose(1, 2).reshape(b, t, hidden)
    x = x + a @ w["o_proj"].T
    h = norm(x, w["post_attention_layernorm"])
    return x + (torch.nn.functional.silu(h @ w["gate_proj"].T) * (h @ w["up_proj"].T)) @ w["down_proj"].T


def test_fused_form_equals_module_sequence():
    w, fused = make(fused=True)
    _, plain = make(fused=False)
    x = torch.randn(2, 37, 512, generator=torch.Generator().manual_seed(1)).half().cuda()
    cos, sin = rotary_tables(torch.arange(37, device="cuda"), 128)
    y1, (k1, v1) = fused(x, cos, sin)
    y2, (k2, v2) = plain(x, cos, sin)
    assert torch.equal(k1, k2) and torch.equal(v1, v2)
    # the RMSNorm prologue of the fused form may differ from torch's in the last float32 bit of a few values
    diff = (y1.float() - y2.float()).abs()
    assert (diff > 0).float().mean() < 0.05 and diff.max() < 0.05 * y2.float().abs().max()


def test_decoding_with_the_cache_matches_prefill():
    _, layer = make(seed=3)
    t = 9
    x = torch.randn(1, t, 512, generator=torch.Generator().manual_seed(2)).half().cuda()
    cos, sin = rotary_tables(torch.arange(t, device="cuda"), 128)
    full, _ = layer(x, cos, sin)
    cache, outs = None, []
    for i in range(t):
        y, cache = layer(x[:, i:i + 1], cos[i:i + 1], sin[i:i + 1], cache)
        outs.append(y)
    step = torch.cat(outs, dim=1)
    assert cache[0].shape == (1, 2, t, 128)
    # same quantised operands in front of attention token by token; the attention arithmetic differs between the two
    # shapes (fused kernel / batched matrix products) in the last fp16 bits, which the o_proj quantiser can turn into a
    # flipped code here and there: equal within the quantisation noise, token 0 (no past) bit for bit
    assert torch.equal(step[:, 0], full[:, 0])
    rel = (step.float() - full.float()).norm(dim=-1) / full.float().norm(dim=-1)
    assert float(rel.max()) < 0.1 and float(rel.median()) < 0.02, rel


def test_close_to_the_fp16_layer():
    w, layer = make(seed=5)
    x = torch.randn(2, 64, 512, generator=torch.Generator().manual_seed(4)).half().cuda()
    cos, sin = rotary_tables(torch.arange(64, device="cuda"), 128)
    got, _ = layer(x, cos, sin)
    want = fp16_layer(w, x, cos, sin, 4, 2)
    err = (got.float() - want.float()).norm() / (want.float() - x.float()).norm()
    print(f"relative error of the layer's update against fp16: {err:.3f}", flush=True)
    assert err < 0.6       # two W4A4 linears in sequence on Gaussian data: ~0.16 each, amplified by the MLP product


def test_token_configuration():
    """Whole-row online rotation + per-token scales, weights rotated offline with per-channel scales (hidden 4096 and
    intermediate 11008 = 172 x 64, the sizes the rotation kernels are built for): close to the fp16 layer, closer
    than the unrotated group configuration on activations with outlier channels, and the fused form (RMSNorm
    inside the rotation kernel, shared launches) agrees with the module sequence."""
    dims = dict(hidden=4096, heads=32, kv_heads=32, inter=11008)
    w, token = make(seed=7, activation="token", **dims)
    _, plain = make(seed=7, activation="token", fused=False, **dims)
    _, group = make(seed=7, activation="group", **dims)
    x = torch.randn(1, 48, 4096, generator=torch.Generator().manual_seed(8)).half().cuda()
    x[..., ::97] *= 12.0                                 # outlier channels
    cos, sin = rotary_tables(torch.arange(48, device="cuda"), 128)
    want = fp16_layer(w, x, cos, sin, 32, 32)
    upd = (want.float() - x.float()).norm()
    err = {name: ((layer(x, cos, sin)[0].float() - want.float()).norm() / upd).item()
           for name, layer in (("token", token), ("token, module sequence", plain), ("group", group))}
    print({k: round(v, 3) for k, v in err.items()}, flush=True)
    assert err["token"] < 0.5 and abs(err["token"] - err["token, module sequence"]) < 0.05
    assert err["token"] < err["group"]


def test_six_bit_layer_gives_the_same_bits():
    w, _ = make(seed=9)
    plain = W4A4DecoderLayer.from_float(w, 4, 2, six_bit=False)
    six = W4A4DecoderLayer.from_float(w, 4, 2, six_bit=True)
    x = torch.randn(1, 300, 512, generator=torch.Generator().manual_seed(10)).half().cuda()
    cos, sin = rotary_tables(torch.arange(300, device="cuda"), 128)
    a, (ka, va) = plain(x, cos, sin)
    b, (kb, vb) = six(x, cos, sin)
    assert six.q_proj._w6 is not None and six.down_proj._w6 is not None     # the 6-bit path really ran
    assert plain.q_proj._w6 is None and plain.down_proj._w6 is None
    assert torch.equal(a, b) and torch.equal(ka, kb) and torch.equal(va, vb)


@pytest.mark.parametrize("six", [None, True])
def test_token_layer_on_the_six_bit_path_gives_the_same_bits(six):
    """Token configuration with group-scaled weights (the Llama-3 arrangement): from 256 rows on the layer's quantisers
    write the 6-bit operand format directly and the linears run on the 6-bit matrix instruction (`six_bit=None`, the
    automatic setting: for group-scaled weights); outputs and cached keys / values must equal the int8 path's bit for bit."""
    w, _ = make(seed=21)
    group = 128 if six is None else 0                 # per-channel scales take the 6-bit path only when asked to
    plain = W4A4DecoderLayer.from_float(w, 4, 2, activation="token", weight_group_size=group, six_bit=False)
    fast = W4A4DecoderLayer.from_float(w, 4, 2, activation="token", weight_group_size=group, six_bit=six)
    x = torch.randn(2, 150, 512, generator=torch.Generator().manual_seed(22)).half().cuda()
    cos, sin = rotary_tables(torch.arange(150, device="cuda"), 128)
    a, (ka, va) = plain(x, cos, sin)
    b, (kb, vb) = fast(x, cos, sin)
    assert fast.q_proj._w6 is not None and fast.o_proj._w6 is not None and fast.down_proj._w6 is not None
    assert plain.q_proj._w6 is None
    assert torch.equal(ka, kb) and torch.equal(va, vb)
    assert torch.equal(a, b)
    short = x[:, :8].contiguous()                     # 16 rows: below the threshold, the int8 / decode kernels
    cs, ss = rotary_tables(torch.arange(8, device="cuda"), 128)
    assert torch.equal(plain(short, cs, ss)[0], fast(short, cs, ss)[0])


def test_fast_rotation_option_changes_almost_nothing():
    """fast_rotation=True: rows of 4096 channels rotate on the matrix cores in the fused prefill path.  Codes differ from the
    float32-butterfly launches in fewer than 1e-4 of the values (tests/test_gpu_rotate_f6.py), so the layer's update moves
    by far less than its int4 noise; the decode path (a single token) stays on the bit-exact kernels."""
    import math
    from flh_amd.quantized_model import W4A4DecoderLayer, rotary_tables
    torch.manual_seed(3)
    hidden, inter, heads = 4096, 1024, 32
    dims = {"q_proj": (hidden, hidden), "k_proj": (hidden, hidden), "v_proj": (hidden, hidden), "o_proj": (hidden, hidden),
            "gate_proj": (inter, hidden), "up_proj": (inter, hidden), "down_proj": (hidden, inter)}
    w = {n: (torch.randn(s, device="cuda") / math.sqrt(s[1])).half() for n, s in dims.items()}
    for six in (False, None):
        layer = W4A4DecoderLayer.from_float(w, heads, heads, fused=True, activation="token", weight_group_size=128, six_bit=six)
        x = torch.randn(2, 160, hidden, device="cuda").half()
        cos, sin = rotary_tables(torch.arange(160, device="cuda"), 128)
        print(f"case layer fast rotation six_bit={six}", flush=True)
        with torch.no_grad():
            y0, (k0, v0) = layer(x, cos, sin)
            layer.fast_rotation = True
            y1, (k1, v1) = layer(x, cos, sin)
            rel = ((y1.float() - y0.float()).norm() / (y0.float() - x.float()).norm()).item()
            print(f"  relative difference of the layer's update {rel:.2e}", flush=True)
            assert 0 < rel < 2e-2
            # one token: the same launches with or without the option
            d1, _ = layer(x[:, :1].contiguous(), cos[:1], sin[:1])
            layer.fast_rotation = False
            d0, _ = layer(x[:, :1].contiguous(), cos[:1], sin[:1])
            assert torch.equal(d0, d1)
