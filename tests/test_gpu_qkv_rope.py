"""flh_gemm_i4_qkv_rope_o16 -- the q / k / v GEMM whose epilogue applies the rotary embedding and writes the key / value
cache -- against the two launches it replaces: the oracle GEMM's fp16 outputs pushed through the tensor expression
q * cos + rotate_half(q) * sin in fp16 (the roundings of flh_rope_kv_cache_f16, pinned by its own test), bit for bit, for
every scale layout and tile, ragged token counts, grouped queries, scattered cache slots and a slot outside the cache."""
import numpy as np
import pytest
import torch

from flh_amd import synthetic as syn

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    import flh_amd
    return flh_amd._CUDA


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def rot_half(x):
    h = x.size(-1) // 2
    return torch.cat((-x[..., h:], x[..., :h]), dim=-1)


def case(batch, t, hq, hkv, k, seed, a_cols, b_cols):
    rng = np.random.default_rng(seed)
    m, ng = batch * t, k // 128
    ap = syn.pack_codes(rng.integers(-8, 8, size=(m, k), dtype=np.int8))
    sa = rng.uniform(0.01, 0.1, size=(m, ng if a_cols > 1 else 1)).astype(np.float16)
    ws, ss = [], []
    for i, n in enumerate((hq * 128, hkv * 128, hkv * 128)):
        ws.append(syn.pack_codes(rng.integers(-8, 8, size=(n, k), dtype=np.int8)))
        ss.append(syn.weight_scales(n, ng if b_cols > 1 else 1, seed + 1 + i))
    return ap, sa, ws, ss


def run(ops, batch, t, hq, hkv, k, seed, a_cols, b_cols, max_len=None, bad_slot=False):
    from flh_amd.quantized_model import rotary_tables
    from oracle import gemm as G
    ap, sa, ws, ss = case(batch, t, hq, hkv, k, seed, a_cols, b_cols)
    max_len = max_len or t + 9
    gen = torch.Generator(device="cuda").manual_seed(seed)
    pos = torch.randperm(max_len, device="cuda", generator=gen)[:t].contiguous()
    if bad_slot:
        pos[t // 2] = max_len + 3                     # outside the cache: that token's key / value are not written
    cos, sin = rotary_tables(pos.clamp(max=max_len - 1), 128, 10000.0)
    kc = torch.full((batch, hkv, max_len, 128), 7.0, dtype=torch.float16, device="cuda")
    vc = torch.full_like(kc, -3.0)
    q = ops.gemm_i4_qkv_rope(dev(ap), dev(sa), [dev(w) for w in ws], [dev(s) for s in ss], cos, sin, pos, kc, vc, batch)
    assert q.shape == (batch, t, hq, 128)
    # expected: oracle GEMMs (fp16), then the fp16 tensor expression
    outs = [dev(G.gemm_i4_dequant(ap, w, sa, s, 128)[0]) for w, s in zip(ws, ss)]
    q0 = outs[0].view(batch, t, hq, 128)
    k0 = outs[1].view(batch, t, hkv, 128)
    v0 = outs[2].view(batch, t, hkv, 128)
    c4, s4 = cos[None, :, None, :], sin[None, :, None, :]
    assert torch.equal(q, q0 * c4 + rot_half(q0) * s4)
    k_want = (k0 * c4 + rot_half(k0) * s4).transpose(1, 2)
    ok = pos < max_len
    assert torch.equal(kc[:, :, pos[ok]], k_want[:, :, ok]) and torch.equal(vc[:, :, pos[ok]], v0.transpose(1, 2)[:, :, ok])
    untouched = torch.ones(max_len, dtype=torch.bool, device="cuda")
    untouched[pos[ok]] = False
    assert bool((kc[:, :, untouched] == 7.0).all()) and bool((vc[:, :, untouched] == -3.0).all())
    return q, kc, vc


@pytest.mark.parametrize("batch,t,hq,hkv,k", [(1, 70, 4, 4, 256), (3, 50, 4, 2, 512), (2, 300, 8, 2, 384), (8, 64, 8, 8, 256),
                                              (1, 5, 2, 1, 128)])
@pytest.mark.parametrize("scales", ["row", "token_group", "group_group"])
def test_qkv_rope_gemm_against_the_oracle(ops, batch, t, hq, hkv, k, scales):
    a_cols, b_cols = {"row": (1, 1), "token_group": (1, 2), "group_group": (2, 2)}[scales]
    print(f"case qkv rope batch={batch} t={t} hq={hq} hkv={hkv} k={k} {scales}", flush=True)
    run(ops, batch, t, hq, hkv, k, batch + t + k, a_cols, b_cols)


@pytest.mark.parametrize("tile", [256, 128])
def test_qkv_rope_gemm_every_tile(ops, tile, gemm_tuning):
    print(f"case qkv rope tile={tile}", flush=True)
    gemm_tuning(tile)
    forced = run(ops, 2, 300, 8, 2, 640, 11, 1, 1)
    gemm_tuning(0)
    auto = run(ops, 2, 300, 8, 2, 640, 11, 1, 1)
    for a, b in zip(forced, auto):
        assert torch.equal(a, b)


def test_qkv_rope_gemm_slot_outside_the_cache(ops):
    print("case qkv rope bad slot", flush=True)
    run(ops, 2, 40, 4, 2, 256, 3, 1, 1, bad_slot=True)


def test_qkv_rope_gemm_equals_the_two_launches_at_llama_width(ops):
    """4096 -> 32 / 8 heads at 4 x 128 tokens: the fused launch against gemm_i4_dequant_multi + rope_kv_cache_."""
    from flh_amd.quantized_model import rotary_tables
    print("case qkv rope llama width", flush=True)
    batch, t, hq, hkv, k = 4, 128, 32, 8, 4096
    ap, sa, ws, ss = case(batch, t, hq, hkv, k, 21, 1, 2)
    A, S, W, WS = dev(ap), dev(sa), [dev(w) for w in ws], [dev(s) for s in ss]
    pos = torch.arange(5, 5 + t, device="cuda")
    cos, sin = rotary_tables(pos, 128, 500000.0)
    kc, vc = (torch.zeros(batch, hkv, 160, 128, dtype=torch.float16, device="cuda") for _ in range(2))
    q = ops.gemm_i4_qkv_rope(A, S, W, WS, cos, sin, pos, kc, vc, batch)
    q2, k2, v2 = ops.gemm_i4_dequant_multi(A, W, S, WS, 128)
    kc2, vc2 = torch.zeros_like(kc), torch.zeros_like(vc)
    q2 = q2.view(batch, t, hq, 128)
    ops.rope_kv_cache_(q2, k2.view(batch, t, hkv, 128), v2.view(batch, t, hkv, 128), cos, sin, pos, kc2, vc2)
    assert torch.equal(q, q2) and torch.equal(kc, kc2) and torch.equal(vc, vc2)


@pytest.mark.parametrize("batch,t,hq,hkv,k", [(1, 70, 4, 4, 256), (3, 50, 4, 2, 512), (2, 300, 8, 2, 384), (1, 5, 2, 1, 128)])
@pytest.mark.parametrize("scales", ["row", "token_group", "group_group"])
@pytest.mark.parametrize("tile", [0, 256])                         # 256: the eight-wave tile of the row-scale launch
def test_qkv_rope_gemm_on_the_six_bit_instruction(ops, batch, t, hq, hkv, k, scales, tile, gemm_tuning):
    """flh_gemm_f6_qkv_rope_o16: the same queries and cache bytes as the int8 launch (itself checked against the oracle)."""
    from flh_amd.quantized_model import rotary_tables
    a_cols, b_cols = {"row": (1, 1), "token_group": (1, 2), "group_group": (2, 2)}[scales]
    print(f"case qkv rope f6 batch={batch} t={t} hq={hq} hkv={hkv} k={k} {scales}", flush=True)
    ap, sa, ws, ss = case(batch, t, hq, hkv, k, batch + t + k + 7, a_cols, b_cols)
    A, S, W, WS = dev(ap), dev(sa), [dev(w) for w in ws], [dev(s) for s in ss]
    max_len = t + 11
    pos = torch.randperm(max_len, device="cuda", generator=torch.Generator(device="cuda").manual_seed(3))[:t].contiguous()
    cos, sin = rotary_tables(pos, 128, 10000.0)
    kc = torch.full((batch, hkv, max_len, 128), 7.0, dtype=torch.float16, device="cuda")
    vc = torch.full_like(kc, -3.0)
    kc6, vc6 = kc.clone(), vc.clone()
    q = ops.gemm_i4_qkv_rope(A, S, W, WS, cos, sin, pos, kc, vc, batch)
    gemm_tuning(tile)
    q6 = ops.gemm_f6_qkv_rope(ops.encode_f6(A), S, [ops.encode_f6(w) for w in W], WS, cos, sin, pos, kc6, vc6, batch)
    gemm_tuning(0)
    assert torch.equal(q, q6) and torch.equal(kc, kc6) and torch.equal(vc, vc6)


def test_qkv_rope_gemm_argument_checks(ops):
    ap, sa, ws, ss = case(1, 70, 4, 4, 256, 1, 1, 1)
    pos = torch.arange(70, device="cuda")
    cos = torch.ones(70, 128, device="cuda").half()
    kc = torch.zeros(1, 4, 80, 128, dtype=torch.float16, device="cuda")
    args = (dev(ap), dev(sa), [dev(w) for w in ws], [dev(s) for s in ss])
    with pytest.raises(RuntimeError):
        ops.gemm_i4_qkv_rope(*args, cos[:, :64].contiguous(), cos, pos, kc, kc.clone(), 1)
    with pytest.raises(RuntimeError):
        ops.gemm_i4_qkv_rope(*args, cos, cos, pos.int(), kc, kc.clone(), 1)
    with pytest.raises(RuntimeError):
        ops.gemm_i4_qkv_rope(*args, cos, cos, pos, kc[:, :2].contiguous(), kc.clone(), 1)
    with pytest.raises(RuntimeError):
        ops.gemm_i4_qkv_rope(*args, cos, cos, pos, kc, kc.clone(), 3)
