"""flh_rope_kv_cache_f16 -- rotary embedding of q / k and the cache write in one launch -- against the tensor
expression it replaces (bit for bit: the same fp16 roundings op by op) and against the float64 oracle (one rounding
instead of three: at most two fp16 steps apart)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def rot_half(x):
    h = x.size(-1) // 2
    return torch.cat((-x[..., h:], x[..., :h]), dim=-1)


@pytest.mark.parametrize("b,t,hq,hkv,d", [(1, 1, 32, 8, 128), (16, 1, 32, 8, 128), (2, 37, 4, 2, 64), (3, 5, 8, 8, 128),
                                           (2, 19, 6, 3, 96), (1, 33, 5, 1, 80), (2, 7, 3, 3, 144)])
@pytest.mark.parametrize("route", ["ext", "ctypes"])
def test_rope_and_cache_write(b, t, hq, hkv, d, route):
    import flh_amd
    from flh_amd import _ops
    from flh_amd.quantized_model import rotary_tables
    from oracle import layer as OL
    ops = flh_amd._CUDA if route == "ext" else _ops
    gen = torch.Generator(device="cuda").manual_seed(b * 100 + t)
    q = torch.randn(b, t, hq, d, device="cuda", generator=gen).half()
    k = torch.randn(b, t, hkv, d, device="cuda", generator=gen).half()
    v = torch.randn(b, t, hkv, d, device="cuda", generator=gen).half()
    max_len = 64
    pos = (torch.randperm(max_len, device="cuda", generator=gen)[:t]).contiguous()
    cos, sin = rotary_tables(pos, d, 500000.0)
    kc = torch.full((b, hkv, max_len, d), 7.0, dtype=torch.float16, device="cuda")
    vc = torch.full_like(kc, -3.0)
    print(f"case rope b={b} t={t} hq={hq} hkv={hkv} d={d} {route}", flush=True)
    c4, s4 = cos[None, :, None, :], sin[None, :, None, :]
    q_want = q * c4 + rot_half(q) * s4
    k_want = k * c4 + rot_half(k) * s4
    q0 = q.clone()
    out = ops.rope_kv_cache_(q, k, v, cos, sin, pos, kc, vc)
    assert out.data_ptr() == q.data_ptr()
    assert torch.equal(q, q_want)
    assert torch.equal(kc[:, :, pos], k_want.transpose(1, 2)) and torch.equal(vc[:, :, pos], v.transpose(1, 2))
    untouched = torch.ones(max_len, dtype=torch.bool, device="cuda")
    untouched[pos] = False
    assert bool((kc[:, :, untouched] == 7.0).all()) and bool((vc[:, :, untouched] == -3.0).all())
    # float64 oracle: [B, H, T, d] layout
    ref = OL.apply_rotary(q0.transpose(1, 2).cpu().numpy(), cos.cpu().numpy(), sin.cpu().numpy())
    got = q.transpose(1, 2).cpu().numpy()
    assert np.abs(got.astype(np.float64) - ref.astype(np.float64)).max() <= 2 * 2.0 ** -10 * np.abs(ref.astype(np.float64)).max()


def test_rope_cache_position_out_of_range_writes_nothing_and_errors():
    import flh_amd
    ops = flh_amd._CUDA
    q = torch.randn(1, 2, 4, 64, device="cuda").half()
    k = torch.randn(1, 2, 2, 64, device="cuda").half()
    v = torch.randn(1, 2, 2, 64, device="cuda").half()
    cos = torch.ones(2, 64, device="cuda").half()
    sin = torch.zeros(2, 64, device="cuda").half()
    kc = torch.zeros(1, 2, 8, 64, dtype=torch.float16, device="cuda")
    vc = torch.zeros_like(kc)
    q0 = q.clone()
    ops.rope_kv_cache_(q, k, v, cos, sin, torch.tensor([3, 99], device="cuda"), kc, vc)
    assert torch.equal(q, q0)                                   # cos = 1, sin = 0: the identity
    assert torch.equal(kc[0, :, 3], k[0, 0]) and int(kc.count_nonzero()) == int(k[0, 0].count_nonzero())
    with pytest.raises(RuntimeError):
        ops.rope_kv_cache_(q, k, v, cos[:1], sin[:1], torch.tensor([3, 4], device="cuda"), kc, vc)
    with pytest.raises(RuntimeError):
        ops.rope_kv_cache_(q, k, v, cos, sin, torch.tensor([3, 4], device="cuda", dtype=torch.int32), kc, vc)
