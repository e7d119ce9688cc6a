"""flh_prefill_attention_f16 -- causal attention of a block of new tokens over the key / value cache -- against the
float64 oracle (oracle/layer.attention_f64, pinned by tests/test_oracle_layer.py): ragged block lengths, a cache that
already holds earlier tokens, grouped queries, batches, garbage in the cache slots no query may see.  Tolerance: the
probabilities are rounded to fp16 before the second product (relative 2^-11 each) and the result once more, so
|error| <= 2e-3 * max|v| + one fp16 step; a wrong mask, head mapping or key order would be O(1)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def run(b, t, hq, hkv, past, seed, max_len=None, scale=None):
    import flh_amd
    from oracle import layer as OL
    ops = flh_amd._CUDA
    gen = torch.Generator(device="cuda").manual_seed(seed)
    max_len = max_len or past + t + 5
    q = torch.randn(b, t, hq, 128, device="cuda", generator=gen).half()
    kc = torch.randn(b, hkv, max_len, 128, device="cuda", generator=gen).half()
    vc = torch.randn(b, hkv, max_len, 128, device="cuda", generator=gen).half()
    kc[:, :, past + t:] = 300.0                      # slots nobody may see: huge scores if the mask slips
    vc[:, :, past + t:] = float("nan")
    out = ops.prefill_attention(q, kc, vc, past, scale)
    assert out.shape == (b, t, hq * 128) and out.dtype == torch.float16
    n = past + t
    qh = q.transpose(1, 2).cpu().numpy()
    if scale is not None:                            # the oracle divides by sqrt(d): fold another scale into q (exact for powers of two)
        qh = (qh.astype(np.float32) * (scale * np.sqrt(128.0))).astype(np.float16)
    ref = OL.attention_f64(qh, kc[:, :, :n].cpu().numpy(), vc[:, :, :n].cpu().numpy(), past)
    got = out.view(b, t, hq, 128).transpose(1, 2).cpu().numpy()
    assert np.isfinite(got.astype(np.float32)).all()
    err = np.abs(got.astype(np.float64) - ref.astype(np.float64)).max()
    assert err <= 2e-3 * float(vc[:, :, :n].abs().max()) + 2.0 ** -10, err
    return out


@pytest.mark.parametrize("b,t,hq,hkv,past", [(1, 1, 4, 4, 0), (1, 31, 4, 2, 0), (2, 64, 8, 2, 0), (1, 128, 4, 4, 0),
                                             (1, 129, 8, 1, 0), (2, 300, 4, 4, 0), (1, 512, 8, 8, 0), (3, 70, 8, 2, 37),
                                             (1, 200, 4, 1, 129), (2, 5, 4, 4, 600), (1, 1, 8, 2, 255)])
def test_prefill_attention_against_the_oracle(b, t, hq, hkv, past):
    print(f"case prefill attention b={b} t={t} hq={hq} hkv={hkv} past={past}", flush=True)
    run(b, t, hq, hkv, past, b * 1000 + t + past)


def test_prefill_attention_with_another_scale():
    print("case prefill attention scale", flush=True)
    run(1, 150, 4, 2, 10, 5, scale=0.125 * 128 ** -0.5 * 8)


def test_prefill_attention_rows_are_independent_of_later_tokens():
    """The causal prefix property on the device: the first 100 outputs of a 260-token block are those of the 100-token
    block, bit for bit (same keys in the same order in the same key blocks)."""
    import flh_amd
    ops = flh_amd._CUDA
    print("case prefill attention prefix", flush=True)
    gen = torch.Generator(device="cuda").manual_seed(9)
    q = torch.randn(1, 260, 4, 128, device="cuda", generator=gen).half()
    kc = torch.randn(1, 2, 300, 128, device="cuda", generator=gen).half()
    vc = torch.randn(1, 2, 300, 128, device="cuda", generator=gen).half()
    full = ops.prefill_attention(q, kc, vc, 20)
    part = ops.prefill_attention(q[:, :100].contiguous(), kc, vc, 20)
    assert torch.equal(full[:, :100], part)


def test_prefill_attention_llama_shape_against_torch():
    """32 / 8 heads, 2 x 1024 tokens: against torch's fused attention on the same fp16 inputs (both within fp16 noise of
    the exact result; the oracle would take minutes at this size)."""
    import flh_amd
    ops = flh_amd._CUDA
    print("case prefill attention llama shape", flush=True)
    gen = torch.Generator(device="cuda").manual_seed(4)
    b, t, hq, hkv = 2, 1024, 32, 8
    q = torch.randn(b, t, hq, 128, device="cuda", generator=gen).half()
    kc = torch.randn(b, hkv, t, 128, device="cuda", generator=gen).half()
    vc = torch.randn(b, hkv, t, 128, device="cuda", generator=gen).half()
    out = ops.prefill_attention(q, kc, vc, 0).view(b, t, hq, 128)
    ref = torch.nn.functional.scaled_dot_product_attention(q.transpose(1, 2).float(), kc.float().repeat_interleave(4, 1),
                                                           vc.float().repeat_interleave(4, 1), is_causal=True)
    err = (out.transpose(1, 2).float() - ref).abs().max().item()
    assert err <= 2e-3 * vc.abs().max().item() + 2.0 ** -10, err


def test_prefill_attention_argument_checks():
    import flh_amd
    ops = flh_amd._CUDA
    q = torch.zeros(1, 4, 4, 128, dtype=torch.float16, device="cuda")
    kc = torch.zeros(1, 2, 8, 128, dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError):
        ops.prefill_attention(q, kc, kc, 5)                       # past + T exceeds the cache
    with pytest.raises(RuntimeError):
        ops.prefill_attention(q[..., :64].contiguous(), kc[..., :64].contiguous(), kc[..., :64].contiguous(), 0)
    with pytest.raises(RuntimeError):
        ops.prefill_attention(q, torch.zeros(1, 3, 8, 128, dtype=torch.float16, device="cuda"),
                              torch.zeros(1, 3, 8, 128, dtype=torch.float16, device="cuda"), 0)
