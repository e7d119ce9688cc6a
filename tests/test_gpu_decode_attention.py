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
    need = _ops.gemm_i4_workspace_bytes if False else None
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
