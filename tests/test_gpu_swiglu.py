"""The gate / up GEMM that stores only fp16(fp16(silu(gate)) * up) (flh_gemm_i4_swiglu_o16) against the oracle:
gate and up from the oracle GEMM (bit-exact fp16, as the separate launches store them) combined by
oracle/prologue.silu_mul_f16.  The exponential and reciprocal are the device's, so the fp16 product may differ from the
float64-exp oracle in its last bit in a few values per thousand; everything else is exact, which the second check pins:
quantising the fused output gives exactly the codes and scales of the separate GEMMs followed by the fused
silu-mul-quantise kernel (same device function on the same fp16 gate / up values)."""
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


def host(t):
    return t.detach().cpu().numpy()


def ulps(a, b):
    """distance in fp16 steps for values of equal sign (a last-bit difference is 1)"""
    ia, ib = a.view(np.int16).astype(np.int32), b.view(np.int16).astype(np.int32)
    return np.abs(ia - ib)


def case(m, n, k, seed, a_cols, b_cols, group=128):
    rng = np.random.default_rng(seed)
    ap = syn.pack_codes(rng.integers(-8, 8, size=(m, k), dtype=np.int8))
    bg = syn.pack_codes(rng.integers(-8, 8, size=(n, k), dtype=np.int8))
    bu = syn.pack_codes(rng.integers(-8, 8, size=(n, k), dtype=np.int8))
    ng = k // group
    sa = rng.uniform(0.01, 0.1, size=(m, ng if a_cols > 1 else 1)).astype(np.float16)
    sg = syn.weight_scales(n, ng if b_cols > 1 else 1, seed + 1)
    su = syn.weight_scales(n, ng if b_cols > 1 else 1, seed + 2)
    return ap, bg, bu, sa, sg, su


def check(ops, m, n, k, seed, a_cols, b_cols):
    from oracle import gemm as G
    from oracle import prologue
    ap, bg, bu, sa, sg, su = case(m, n, k, seed, a_cols, b_cols)
    d = host(ops.gemm_i4_swiglu(dev(ap), dev(bg), dev(bu), dev(sa), dev(sg), dev(su), 128))
    gate, _ = G.gemm_i4_dequant(ap, bg, sa, sg)
    up, _ = G.gemm_i4_dequant(ap, bu, sa, su)
    ref = prologue.silu_mul_f16(gate, up)
    assert d.shape == (m, n)
    differ = d.view(np.uint16) != ref.view(np.uint16)
    assert differ.mean() < 3e-3, differ.mean()
    assert ulps(d[differ], ref[differ]).max(initial=0) <= 2     # one step of fp16(silu) can move the product by two
    return d, gate, up


@pytest.mark.parametrize("m,n,k", [(65, 64, 256), (300, 264, 1024), (130, 1000, 512), (2048, 1408, 512), (1024, 704, 384),
                                   (70, 36, 128)])
@pytest.mark.parametrize("scales", ["row", "token_group", "group_group"])
def test_swiglu_gemm_against_the_oracle(ops, m, n, k, scales):
    a_cols, b_cols = {"row": (1, 1), "token_group": (1, 2), "group_group": (2, 2)}[scales]
    print(f"case swiglu m={m} n={n} k={k} {scales}", flush=True)
    check(ops, m, n, k, m + n + k, a_cols, b_cols)


@pytest.mark.parametrize("tile", [256, 128, 64])
def test_swiglu_gemm_every_tile(ops, tile, gemm_tuning):
    gemm_tuning(tile)
    print(f"case swiglu tile={tile}", flush=True)
    outs = [check(ops, 300, 264, 1408, 5, *cols)[0] for cols in ((1, 1), (1, 2))]
    gemm_tuning(0)
    auto = [check(ops, 300, 264, 1408, 5, *cols)[0] for cols in ((1, 1), (1, 2))]
    for a, b in zip(outs, auto):
        assert np.array_equal(a.view(np.uint16), b.view(np.uint16))       # every tile shape: the same bits


@pytest.mark.parametrize("n,k,b_cols", [(11008, 4096, 1), (14336, 4096, 2)])
def test_swiglu_gemm_full_width_equals_the_separate_launches(ops, n, k, b_cols):
    """Llama-2 / Llama-3 gate-up shapes at M = 2048: the fused launch quantised by the group quantiser gives exactly the
    codes and scales of the two separate GEMMs followed by the silu-mul-quantise kernel (the same device arithmetic on
    the same fp16 gate / up values), and sampled rows agree with the oracle."""
    from oracle import gemm as G
    from oracle import prologue
    m = 2048
    ap, bg, bu, sa, sg, su = case(m, n, k, n, 1, b_cols)
    A, Bg, Bu, Sa, Sg, Su = (dev(v) for v in (ap, bg, bu, sa, sg, su))
    print(f"case swiglu full width n={n} k={k}", flush=True)
    d = ops.gemm_i4_swiglu(A, Bg, Bu, Sa, Sg, Su, 128)
    gate, up = ops.gemm_i4_dequant(A, Bg, Sa, Sg, 128), ops.gemm_i4_dequant(A, Bu, Sa, Su, 128)
    q1, s1 = ops.quant_and_pack_i4(d.view(-1, 128))
    q2, s2 = ops.silu_mul_and_quantize_i4_gs(gate, up, 128)
    assert torch.equal(q1.view(-1), q2.view(-1)) and torch.equal(s1.view(-1), s2.view(-1))
    rows = np.random.default_rng(1).choice(m, 16, replace=False)
    g_ref, _ = G.gemm_i4_dequant(ap[rows], bg, sa[rows], sg)
    u_ref, _ = G.gemm_i4_dequant(ap[rows], bu, sa[rows], su)
    ref = prologue.silu_mul_f16(g_ref, u_ref)
    got = host(d)[rows]
    differ = got.view(np.uint16) != ref.view(np.uint16)
    assert differ.mean() < 3e-3 and ulps(got[differ], ref[differ]).max(initial=0) <= 2


def test_swiglu_layer_method_and_errors(ops):
    from flh_amd.nn import LinearFLH
    k, n, m = 512, 192, 70
    ap, bg, bu, sa, sg, su = case(m, n, k, 3, 1, 2)
    gate, up = LinearFLH(k, n, device="cuda"), LinearFLH(k, n, device="cuda")
    gate.w_packed.copy_(dev(bg).view(-1)), gate.w_scale.copy_(dev(sg))
    up.w_packed.copy_(dev(bu).view(-1)), up.w_scale.copy_(dev(su))
    y = LinearFLH.forward_swiglu(gate, up, dev(ap).view(2, 35, -1), dev(sa).view(2, 35, 1))
    assert y.shape == (2, 35, n)
    assert torch.equal(y.view(m, n), ops.gemm_i4_swiglu(dev(ap), dev(bg), dev(bu), dev(sa), dev(sg), dev(su), 128))
    with pytest.raises(ValueError):
        LinearFLH.forward_swiglu(gate, LinearFLH(k, n + 64, device="cuda"), dev(ap), dev(sa))
    with pytest.raises(RuntimeError):
        ops.gemm_i4_swiglu(dev(ap), dev(bg), dev(bu)[:-1], dev(sa), dev(sg), dev(su), 128)


@pytest.mark.parametrize("m,n,k", [(300, 200, 512), (64, 64, 128), (513, 1000, 1024), (2048, 1408, 4096), (130, 36, 384)])
@pytest.mark.parametrize("a_cols,b_cols", [(1, 1), (1, 2), (2, 2)])
@pytest.mark.parametrize("tile", [0, 64, 128, 256])            # 256: the eight-wave tile (one scale per row only)
def test_six_bit_swiglu_gemm_gives_the_int8_launch_bits(ops, gemm_tuning, m, n, k, a_cols, b_cols, tile):
    """flh_gemm_f6_swiglu_o16 on re-encoded operands against flh_gemm_i4_swiglu_o16 on the nibbles: the sums are the same
    integers, the epilogue the same arithmetic, the product the same device routine -- so bit for bit, for every scale
    layout, ragged M and N, every tile."""
    print(f"case f6 swiglu m={m} n={n} k={k} a_cols={a_cols} b_cols={b_cols} tile={tile}", flush=True)
    ap, bg, bu, sa, sg, su = case(m, n, k, 31 + m + n, a_cols, b_cols)
    a, g, u = dev(ap), dev(bg), dev(bu)
    want = ops.gemm_i4_swiglu(a, g, u, dev(sa), dev(sg), dev(su))
    gemm_tuning(tile, 0)
    got = ops.gemm_f6_swiglu(ops.encode_f6(a), ops.encode_f6(g), ops.encode_f6(u), dev(sa), dev(sg), dev(su))
    gemm_tuning(0, 0)
    assert got.shape == (m, n)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    # ... and against the separate 6-bit launches followed by the product kernel
    g6 = ops.gemm_f6_dequant_o16(ops.encode_f6(a), ops.encode_f6(g), dev(sa), dev(sg)) if b_cols == 1 else \
        ops.gemm_f6_dequant_o16_gs(ops.encode_f6(a), ops.encode_f6(g), dev(sa), dev(sg))
    u6 = ops.gemm_f6_dequant_o16(ops.encode_f6(a), ops.encode_f6(u), dev(sa), dev(su)) if b_cols == 1 else \
        ops.gemm_f6_dequant_o16_gs(ops.encode_f6(a), ops.encode_f6(u), dev(sa), dev(su))
    if n % 8 == 0:
        assert torch.equal(got, ops.silu_mul(g6, u6))


def test_six_bit_swiglu_argument_errors(ops):
    a6 = torch.zeros(4, 96, dtype=torch.uint8, device="cuda")
    b6 = torch.zeros(8, 96, dtype=torch.uint8, device="cuda")
    s1 = torch.ones(4, 1, dtype=torch.float16, device="cuda")
    w1 = torch.ones(8, 1, dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError):
        ops.gemm_f6_swiglu(a6, b6, b6[:4].contiguous(), s1, w1, w1)
    with pytest.raises(RuntimeError):
        ops.gemm_f6_swiglu(a6, b6, b6, s1, w1, w1[:4].contiguous())
    with pytest.raises(RuntimeError):
        ops.gemm_f6_swiglu(a6, b6, b6, torch.ones(4, 3, dtype=torch.float16, device="cuda"), w1, w1)
