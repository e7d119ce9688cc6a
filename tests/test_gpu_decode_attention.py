"""flh_decode_attention_f16 (one query token per sequence over a preallocated cache, grouped queries, chunked over the
cached positions) against the float64 attention of oracle/layer.py, including lengths that end inside a chunk, a single
cached position, peaked and flat score distributions, and a workspace that holds garbage."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def reference(q, k, v, kv_len):
    from oracle import layer as OL
    qn = q.cpu().numpy()[:, :, None, :]                               # [B, H, 1, d]
    kn, vn = k.cpu().numpy()[:, :, :kv_len], v.cpu().numpy()[:, :, :kv_len]
    return OL.attention_f64(qn, kn, vn, past=kv_len - 1)[:, :, 0]


@pytest.mark.parametrize("b,hq,hkv,d,kv_len,max_len", [(1, 32, 8, 128, 2048, 2048), (16, 32, 8, 128, 2048, 2048),
                                                       (3, 32, 32, 128, 777, 1024), (2, 8, 4, 64, 65, 128),
                                                       (2, 8, 1, 128, 1, 64), (1, 16, 8, 64, 130, 256)])
def test_decode_attention_against_float64(b, hq, hkv, d, kv_len, max_len):
    from flh_amd import _ops
    gen = torch.Generator(device="cuda").manual_seed(kv_len + b)
    q = torch.randn(b, hq, d, device="cuda", generator=gen).half()
    k = (torch.randn(b, hkv, max_len, d, device="cuda", generator=gen) * 0.5).half()
    v = torch.randn(b, hkv, max_len, d, device="cuda", generator=gen).half()
    k[:, :, kv_len:] = 100.0                                           # slots past kv_len must not be looked at
    v[:, :, kv_len:] = float("nan")
    print(f"case decode attention b={b} hq={hq} hkv={hkv} d={d} kv_len={kv_len}", flush=True)
    ws = torch.full((int(_ops._lib.load().flh_decode_attention_workspace_bytes(b, hq, d, kv_len)) + 64,), 0xFF,
                    dtype=torch.uint8, device="cuda")                  # NaN patterns: nothing may be read before written
    out = _ops.decode_attention(q, k, v, kv_len, workspace=ws)
    ref = reference(q, k, v, kv_len)
    got = out.cpu().numpy().astype(np.float64)
    assert np.isfinite(got).all()
    assert np.abs(got - ref.astype(np.float64)).max() <= 2e-3 * max(1.0, np.abs(ref.astype(np.float64)).max())
    again = _ops.decode_attention(q, k, v, kv_len)                     # the op's own cached workspace
    assert torch.equal(again, out)


def test_decode_attention_peaked_and_flat():
    from flh_amd import _ops
    b, hq, hkv, d, n = 1, 4, 1, 128, 300
    q = torch.zeros(b, hq, d, device="cuda", dtype=torch.float16)
    q[0, :, 0] = 30.0
    k = torch.zeros(b, hkv, n, d, device="cuda", dtype=torch.float16)
    k[0, 0, 123, 0] = 10.0                                             # one key dominates: score 300 / sqrt(128) = 26.5
    v = torch.randn(b, hkv, n, d, device="cuda").half()
    out = _ops.decode_attention(q, k, v, n)
    assert torch.allclose(out[0, 0].float(), v[0, 0, 123].float(), atol=2e-3)
    flat = _ops.decode_attention(torch.zeros_like(q), k, v, n)         # zero query: the mean of the values
    assert torch.allclose(flat[0, 0].float(), v[0, 0].float().mean(0), atol=2e-3)


def test_decode_attention_argument_errors():
    from flh_amd import _ops
    q = torch.zeros(1, 6, 128, device="cuda", dtype=torch.float16)
    k = torch.zeros(1, 2, 16, 128, device="cuda", dtype=torch.float16)
    with pytest.raises(RuntimeError):
        _ops.decode_attention(q, k, k, 8)                              # 3 query heads per key / value head
    q = torch.zeros(1, 4, 128, device="cuda", dtype=torch.float16)
    with pytest.raises(RuntimeError):
        _ops.decode_attention(q, k, k, 17)                             # kv_len beyond the cache
    with pytest.raises(RuntimeError):
        _ops.decode_attention(q, k, k, 8, workspace=torch.zeros(16, dtype=torch.uint8, device="cuda"))


@pytest.mark.parametrize("b,hq,hkv,d,kv_len,max_len,slot", [(1, 32, 8, 128, 2048, 2048, 2047), (16, 32, 8, 128, 2048, 2048, 2047),
                                                            (3, 32, 32, 128, 777, 1024, 776), (2, 8, 4, 64, 65, 128, 64),
                                                            (2, 8, 1, 128, 1, 64, 0), (2, 16, 8, 64, 130, 256, 70),
                                                            (2, 8, 8, 128, 200, 256, 63), (2, 8, 4, 64, 65, 128, 100),
                                                            (1, 32, 8, 128, 100, 256, 255)])
def test_rotary_and_cache_write_inside_attention_give_the_separate_launches_bits(b, hq, hkv, d, kv_len, max_len, slot):
    """flh_decode_attention_rope_f16 against flh_rope_kv_cache_f16 followed by flh_decode_attention_f16 on copies of the
    same cache: the same output, the same cache contents, bit for bit (slot at the end of the live range, at a chunk
    boundary, in the middle -- an overwrite of an older position -- slot 0 of an empty cache, and a slot beyond the
    live range, which is written and not read); q is left alone."""
    from flh_amd import _ops
    from flh_amd.quantized_model.decoder_layer import rotary_tables
    gen = torch.Generator(device="cuda").manual_seed(kv_len + b + slot)
    q = torch.randn(b, hq, d, device="cuda", generator=gen).half()
    k_new = torch.randn(b, hkv, d, device="cuda", generator=gen).half()
    v_new = torch.randn(b, hkv, d, device="cuda", generator=gen).half()
    k = (torch.randn(b, hkv, max_len, d, device="cuda", generator=gen) * 0.5).half()
    v = torch.randn(b, hkv, max_len, d, device="cuda", generator=gen).half()
    k[:, :, kv_len:] = 100.0
    v[:, :, kv_len:] = float("nan")
    k[:, :, slot] = float("nan")                                       # what the slot held before must not be read
    v[:, :, slot] = float("nan")
    pos = torch.tensor([slot], device="cuda")
    cos, sin = rotary_tables(pos, d, 500000.0)
    print(f"case rotary decode attention b={b} hq={hq} hkv={hkv} d={d} kv_len={kv_len} slot={slot}", flush=True)
    # separate launches
    k1, v1, q1 = k.clone(), v.clone(), q.clone()
    _ops.rope_kv_cache_(q1.view(b, 1, hq, d), k_new.view(b, 1, hkv, d), v_new.view(b, 1, hkv, d), cos, sin, pos, k1, v1)
    want = _ops.decode_attention(q1, k1, v1, kv_len)
    # one pair of launches
    k2, v2, q2 = k.clone(), v.clone(), q.clone()
    got = _ops.decode_attention_rope(q2, k_new, v_new, cos, sin, pos, k2, v2, kv_len)
    assert torch.equal(q2, q)
    assert torch.equal(got, want)
    assert torch.equal(k2.view(torch.int16), k1.view(torch.int16)) and torch.equal(v2.view(torch.int16), v1.view(torch.int16))
    ref = reference(q1, k1, v1, kv_len)
    assert np.abs(got.cpu().numpy().astype(np.float64) - ref.astype(np.float64)).max() <= 2e-3 * max(1.0, np.abs(ref).max())


def test_rotary_decode_attention_argument_errors():
    from flh_amd import _ops
    q = torch.zeros(1, 8, 128, device="cuda", dtype=torch.float16)
    kn = torch.zeros(1, 2, 128, device="cuda", dtype=torch.float16)
    k = torch.zeros(1, 2, 16, 128, device="cuda", dtype=torch.float16)
    cs = torch.zeros(1, 128, device="cuda", dtype=torch.float16)
    pos = torch.zeros(1, device="cuda", dtype=torch.int64)
    with pytest.raises(RuntimeError):
        _ops.decode_attention_rope(q, kn[:, :1].contiguous(), kn, cs, cs, pos, k, k.clone(), 4)
    with pytest.raises(RuntimeError):
        _ops.decode_attention_rope(q, kn, kn, cs[:, :64].contiguous(), cs, pos, k, k.clone(), 4)
    with pytest.raises(RuntimeError):
        _ops.decode_attention_rope(q, kn, kn, cs, cs, pos.int(), k, k.clone(), 4)
    with pytest.raises(RuntimeError):
        _ops.decode_attention_rope(q, kn, kn, cs, cs, pos, k, k.clone(), 17)
